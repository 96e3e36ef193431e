// A selective state-space mixer's own kernels: the short causal filter per channel and the scan.
//
// A request's state is one 32-bit row: [ S: inner x state | the filter's last taps - 1 inputs: (taps - 1) x inner ].
// Everything about the step is read on the device (q_start, the sequences' state slots), so a step can be
// recorded.  A sequence without a slot (a padding row of a fixed-shape step) reads zeros and keeps nothing.
//
//   da_conv_causal        y[n, c] = act(b[c] + sum_k w[c, k] * x[n - (K - 1 - k), c]); rows before the portion come
//                         from the state, rows before the sequence are zero (the state starts as zeros)
//   da_conv_state_update  the state's filter part after the step: the last K - 1 inputs of each sequence
//   da_selective_scan     per channel c and state index j, token by token:
//                           dt = softplus(raw[n, c]);  S[c, j] = exp(dt * A[c, j]) * S[c, j] + dt * x[n, c] * B[n, j]
//                           y[n, c] = (sum_j S[c, j] * C[n, j] + D[c] * x[n, c]) * silu(z[n, c])
//                         with A = -exp(A_log) (handed over in 32-bit; times log2(e) for bfloat16 rows), all in 32-bit; the state is read from the slot at the portion's
//                         start and written back at its end.
//   da_scan_chunk_*       the same scan for long portions, cut into chunks that run side by side: each chunk's
//                         own contribution and decay, then the chunks' starting states one after the other, then
//                         every chunk again from its starting state.
#include "common.h"
#include <type_traits>

#define CONV_MAX_TAPS 16
#define SCAN_SPT 16          // state entries a thread keeps
#define SCAN_BLOCK 256
#define SCAN_TOK 32          // tokens whose B and C wait in LDS together
#define SCAN_GROUP 8         // tokens whose own numbers a thread asks for at once
#define SCAN_LDS_STATE 64    // state entries of B and of C that LDS holds a token

template <typename T>
__global__ void conv_causal_kernel(const T* __restrict__ x, int x_ld, const float* __restrict__ state, long state_ld,
                                   int conv_off, const int* __restrict__ state_slots, const int* __restrict__ seq_of_token,
                                   const int* __restrict__ q_start, const void* __restrict__ w, int w_dtype,
                                   const void* __restrict__ b, int b_dtype, int act, T* __restrict__ y, int y_ld, int N,
                                   int C, int K) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)N * C) return;
  const int n = (int)(i / C), c = (int)(i % C);
  const int s = seq_of_token[n];
  const int first = q_start[s];
  const int slot = state_slots[s];
  const float* tail = slot >= 0 ? state + (size_t)slot * state_ld + conv_off : nullptr;   // [K - 1][C], oldest first
  float acc = b ? load_param(b, b_dtype, c) : 0.f;
  for (int k = 0; k < K; ++k) {
    const int back = K - 1 - k;                    // how many tokens before this one
    const int r = n - back;
    float v;
    if (r >= first) v = to_f32(x[(size_t)r * x_ld + c]);
    else v = tail ? tail[(size_t)(K - 1 + (r - first)) * C + c] : 0.f;
    acc = fmaf(load_param(w, w_dtype, (size_t)c * K + k), v, acc);
  }
  from_f32(&y[(size_t)n * y_ld + c], apply_act(acc, act));
}

extern "C" int da_conv_causal(const void* x, int dtype, int x_ld, const float* state, long state_ld, int conv_off,
                              const int* state_slots, const int* seq_of_token, const int* q_start, const void* w,
                              int w_dtype, const void* b, int b_dtype, int act, void* y, int y_ld, int N, int C, int K,
                              void* stream) {
  DA_REQUIRE(N >= 0 && C > 0 && K >= 1 && K <= CONV_MAX_TAPS && x_ld >= C && y_ld >= C, "conv_causal: bad sizes");
  DA_REQUIRE(state_ld >= conv_off + (long)(K - 1) * C && conv_off >= 0, "conv_causal: the state row is too short");
  DA_REQUIRE(act >= DA_ACT_NONE && act <= DA_ACT_LAST, "conv_causal: unknown activation %d", act);
  if (N == 0) return 0;
  const long total = (long)N * C;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(conv_causal_kernel<bf16_t>, dim3(da_ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)x, x_ld, state, state_ld, conv_off, state_slots, seq_of_token, q_start, w, w_dtype, b,
                       b_dtype, act, (bf16_t*)y, y_ld, N, C, K);
  else
    hipLaunchKernelGGL(conv_causal_kernel<float>, dim3(da_ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const float*)x, x_ld, state, state_ld, conv_off, state_slots, seq_of_token, q_start, w, w_dtype, b,
                       b_dtype, act, (float*)y, y_ld, N, C, K);
  DA_CHECK_LAUNCH("conv_causal");
  return 0;
}

// One thread per (sequence, channel): the K - 1 newest inputs, from the step's rows and, for a portion shorter
// than K - 1, from what the state held.  All reads come before the writes.
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ x, int x_ld, float* __restrict__ state, long state_ld,
                                         int conv_off, const int* __restrict__ state_slots,
                                         const int* __restrict__ q_start, int S, int C, int K) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)S * C) return;
  const int s = (int)(i / C), c = (int)(i % C);
  const int slot = state_slots[s];
  if (slot < 0) return;
  const int first = q_start[s], T_ = q_start[s + 1] - first;
  float* tail = state + (size_t)slot * state_ld + conv_off;
  float keep[CONV_MAX_TAPS];
  for (int k = 0; k < K - 1; ++k) {
    const int r = T_ - (K - 1) + k;                // the portion's row that lands at place k (negative: older)
    keep[k] = r >= 0 ? to_f32(x[(size_t)(first + r) * x_ld + c]) : tail[(size_t)(K - 1 + r) * C + c];
  }
  for (int k = 0; k < K - 1; ++k) tail[(size_t)k * C + c] = keep[k];
}

extern "C" int da_conv_state_update(const void* x, int dtype, int x_ld, float* state, long state_ld, int conv_off,
                                    const int* state_slots, const int* q_start, int S, int C, int K, void* stream) {
  DA_REQUIRE(S >= 0 && C > 0 && K >= 1 && K <= CONV_MAX_TAPS && x_ld >= C, "conv_state_update: bad sizes");
  DA_REQUIRE(state_ld >= conv_off + (long)(K - 1) * C && conv_off >= 0, "conv_state_update: the state row is too short");
  if (S == 0 || K == 1) return 0;
  const long total = (long)S * C;
  if (dtype == DA_BF16)
    hipLaunchKernelGGL(conv_state_update_kernel<bf16_t>, dim3(da_ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)x, x_ld, state, state_ld, conv_off, state_slots, q_start, S, C, K);
  else
    hipLaunchKernelGGL(conv_state_update_kernel<float>, dim3(da_ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream,
                       (const float*)x, x_ld, state, state_ld, conv_off, state_slots, q_start, S, C, K);
  DA_CHECK_LAUNCH("conv_state_update");
  return 0;
}

// ln(1 + e^v) and v / (1 + e^-v) with the hardware's exp2, log2 and reciprocal (each within a unit or two in the last
// place of 32 bits; the library's log1pf and expf cost a hundred instructions a token and channel).  For v below -17
// the sum 1 + e^v is 1 and the result 0 instead of e^v < 4e-8: a step size that small moves nothing.
// The 32-bit path (FAST false) keeps the library's functions.
template <bool FAST>
__device__ __forceinline__ float softplus_f32(float v) {
  if (!FAST) return v > 20.f ? v : log1pf(expf(v));
  const float e = __builtin_amdgcn_exp2f(v * 1.4426950408889634f);
  return v > 20.f ? v : 0.6931471805599453f * __builtin_amdgcn_logf(1.0f + e);
}
template <bool FAST>
__device__ __forceinline__ float silu_f32(float v) {
  if (!FAST) return v / (1.0f + expf(-v));
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

// What a scan kernel reads of the step.
struct ScanIn {
  const void* x; int x_ld;            // [N, inner] after the filter
  const float* raw; int raw_ld;       // [N, inner] step sizes before softplus, 32-bit
  const void* bc; int bc_ld;          // [N, >= b_off + state], [N, >= c_off + state]
  int b_off, c_off;
  const void* z; int z_ld;            // [N, inner] the gate's input
  const float* a2;                    // [inner, state]: bfloat16 rows: A log2(e) = -exp(A_log) log2(e), so that a decay
                                      // exp(dt A) is one exp2 of the hardware; 32-bit rows: A itself, and the library's expf
  const void* d; int d_dtype;         // [inner]
};

// L lanes share a channel; lane `sub` of them keeps the state entries sub * SPT .. sub * SPT + SPT - 1.
// MODE 0: the whole portion in order, state from and to the slot.
// MODE 1: a chunk from a zero state: leaves its contribution (end state) and the sum of its step sizes.
// MODE 2: a chunk from a given starting state: writes y.
template <typename T, int MODE>
__global__ void __launch_bounds__(SCAN_BLOCK)
selective_scan_kernel(ScanIn in, float* __restrict__ state, long state_ld, const int* __restrict__ state_slots,
                      const int* __restrict__ q_start, T* __restrict__ y, int y_ld, int inner, int n_state, int L,
                      int chunk, float* __restrict__ chunk_state, float* __restrict__ chunk_dt, int max_chunks) {
  const int s = blockIdx.y;
  const int slot = state_slots[s];
  const int first = q_start[s], len = q_start[s + 1] - first;
  const int k = MODE == 0 ? 0 : blockIdx.z;
  const int t0 = MODE == 0 ? 0 : k * chunk;
  const int t1 = MODE == 0 ? len : (t0 + chunk < len ? t0 + chunk : len);
  if (t0 >= len) return;
  const int g = blockIdx.x * SCAN_BLOCK + threadIdx.x;
  const int c = g / L, sub = g % L;
  const bool live = c < inner;                       // lanes past the last channel follow along and store nothing
  const int cc = live ? c : inner - 1;
  const int j0 = sub * SCAN_SPT;
  // Every load of the prologue is asked for at once, from a place that exists (an entry past the state's end reads
  // the row's first one), and looked at afterwards: a load under a condition would be waited for on the spot.
  float A[SCAN_SPT], S[SCAN_SPT];
  const float* s_from = MODE == 2 ? chunk_state + (((size_t)s * max_chunks + k) * inner + cc) * n_state
                                  : state + (size_t)(slot >= 0 ? slot : 0) * state_ld + (size_t)cc * n_state;
  const bool s_given = MODE == 2 || (MODE == 0 && slot >= 0);
#pragma unroll
  for (int j = 0; j < SCAN_SPT; ++j) {
    const int jj = j0 + j < n_state ? j0 + j : 0;
    A[j] = in.a2[(size_t)cc * n_state + jj];
    S[j] = MODE == 1 ? 0.f : s_from[jj];
  }
#pragma unroll
  for (int j = 0; j < SCAN_SPT; ++j) {
    const bool in_j = j0 + j < n_state;
    A[j] = in_j ? A[j] : 0.f;
    S[j] = (in_j && s_given) ? S[j] : 0.f;
  }
  const float Dc = in.d ? load_param(in.d, in.d_dtype, cc) : 0.f;
  float dt_sum = 0.f;
  // B and C of a token are the same for all channels: groups of SCAN_TOK tokens' B | C wait in LDS (up to
  // SCAN_LDS_STATE entries each; longer ones are read from memory), and the tokens' own numbers (step size, x, gate)
  // are asked for SCAN_GROUP tokens at a time, so that a step of the recurrence does not wait for memory.
  __shared__ __attribute__((aligned(16))) float bcs[SCAN_TOK][2][SCAN_LDS_STATE];
  const bool staged = n_state <= SCAN_LDS_STATE;
  for (int tb = t0; tb < t1; tb += SCAN_TOK) {
    const int nt = t1 - tb < SCAN_TOK ? t1 - tb : SCAN_TOK;
    if (staged) {
      __syncthreads();                                // the group before has been read by everyone
      for (int i = threadIdx.x; i < nt * 2 * n_state; i += SCAN_BLOCK) {
        const int tok = i / (2 * n_state), r = i % (2 * n_state), which = r / n_state, j = r % n_state;
        bcs[tok][which][j] = to_f32(((const T*)in.bc)[((size_t)first + tb + tok) * in.bc_ld + (which ? in.c_off : in.b_off) + j]);
      }
      __syncthreads();
    }
    // a group of tokens' own numbers (step size, x, gate) for this thread's channel, all asked for at once, and the
    // next group's before this group's arithmetic (two sets of registers, taken in turn)
    float raw_g[2][SCAN_GROUP], x_g[2][SCAN_GROUP], z_g[2][SCAN_GROUP];
    auto ask = [&](int tg, auto set) {
      constexpr int b = decltype(set)::value;
#pragma unroll
      for (int u = 0; u < SCAN_GROUP; ++u) {
        const size_t nn = (size_t)first + tb + (tg + u < nt ? tg + u : nt - 1);
        raw_g[b][u] = in.raw[nn * in.raw_ld + cc];
        x_g[b][u] = to_f32(((const T*)in.x)[nn * in.x_ld + cc]);
        z_g[b][u] = MODE != 1 ? to_f32(((const T*)in.z)[nn * in.z_ld + cc]) : 0.f;
      }
    };
    auto group = [&](int tg, auto set) {
      constexpr int b = decltype(set)::value;
      if (tg + SCAN_GROUP < nt) ask(tg + SCAN_GROUP, std::integral_constant<int, 1 - b>{});
      __builtin_amdgcn_sched_barrier(0);              // (asked for here, not where the values are used)
      float y_g[SCAN_GROUP];
#pragma unroll
      for (int u = 0; u < SCAN_GROUP; ++u) {
        const int t = tg + u;
        if (t < nt) {                                 // (the same for every thread of the workgroup)
          const size_t n = (size_t)first + tb + t;
          const float xv = x_g[b][u];
          const float dt = softplus_f32<sizeof(T) == 2>(raw_g[b][u]);
          const float dx = dt * xv;
          float Bv[SCAN_SPT], Cv[SCAN_SPT];
          if (staged) {                               // 16 entries of B and of C in four reads each
#pragma unroll
            for (int q4 = 0; q4 < SCAN_SPT / 4; ++q4) {
              const float4 bq = *(const float4*)&bcs[t][0][j0 + 4 * q4];
              Bv[4 * q4] = bq.x; Bv[4 * q4 + 1] = bq.y; Bv[4 * q4 + 2] = bq.z; Bv[4 * q4 + 3] = bq.w;
              if (MODE != 1) {
                const float4 cq = *(const float4*)&bcs[t][1][j0 + 4 * q4];
                Cv[4 * q4] = cq.x; Cv[4 * q4 + 1] = cq.y; Cv[4 * q4 + 2] = cq.z; Cv[4 * q4 + 3] = cq.w;
              }
            }
          } else {
            const T* bc = (const T*)in.bc + n * in.bc_ld;
#pragma unroll
            for (int j = 0; j < SCAN_SPT; ++j) {
              const int jj = j0 + j < n_state ? j0 + j : 0;
              Bv[j] = to_f32(bc[in.b_off + jj]);
              if (MODE != 1) Cv[j] = to_f32(bc[in.c_off + jj]);
            }
          }
          float part = 0.f;
#pragma unroll
          for (int j = 0; j < SCAN_SPT; ++j) {
            const bool in_j = j0 + j < n_state;
            const float Bj = in_j ? Bv[j] : 0.f;
            S[j] = (sizeof(T) == 2 ? __builtin_amdgcn_exp2f(dt * A[j]) : expf(dt * A[j])) * S[j] + dx * Bj;
            if (MODE != 1) part = fmaf(S[j], in_j ? Cv[j] : 0.f, part);
          }
          dt_sum += dt;
          if (MODE != 1) {
            for (int o = 1; o < L; o <<= 1) part += __shfl_xor(part, o, DA_WAVE);     // the lanes of one channel, fixed order
            y_g[u] = (part + Dc * xv) * silu_f32<sizeof(T) == 2>(z_g[b][u]);
          }
        }
      }
      if (MODE != 1 && live && sub == 0) {            // the group's results leave together, behind its arithmetic
#pragma unroll
        for (int u = 0; u < SCAN_GROUP; ++u)
          if (tg + u < nt) from_f32(&y[((size_t)first + tb + tg + u) * y_ld + cc], y_g[u]);
      }
    };
    ask(0, std::integral_constant<int, 0>{});
    for (int tg = 0; tg < nt; tg += 2 * SCAN_GROUP) {
      group(tg, std::integral_constant<int, 0>{});
      if (tg + SCAN_GROUP < nt) group(tg + SCAN_GROUP, std::integral_constant<int, 1>{});
    }
  }
  if (!live) return;
  if (MODE == 0 && slot >= 0) {
#pragma unroll
    for (int j = 0; j < SCAN_SPT; ++j)
      if (j0 + j < n_state) state[(size_t)slot * state_ld + (size_t)cc * n_state + j0 + j] = S[j];
  }
  if (MODE == 1) {
    float* st = chunk_state + (((size_t)s * max_chunks + k) * inner + cc) * n_state;
#pragma unroll
    for (int j = 0; j < SCAN_SPT; ++j)
      if (j0 + j < n_state) st[j0 + j] = S[j];
    if (sub == 0) chunk_dt[((size_t)s * max_chunks + k) * inner + cc] = dt_sum;
  }
}

// The chunks' starting states, one chunk after the other: start_0 = the slot's state, start_{k+1} =
// exp(A * sum of chunk k's step sizes) * start_k + chunk k's contribution; in place (a chunk's contribution is
// replaced by its starting state), and the state after the last chunk goes back to the slot.
__global__ void scan_chunk_carry_kernel(float* __restrict__ chunk_state, const float* __restrict__ chunk_dt,
                                        int max_chunks, int chunk, float* __restrict__ state, long state_ld,
                                        const int* __restrict__ state_slots, const int* __restrict__ q_start,
                                        const float* __restrict__ a2, int inner, int n_state, int fast) {
  const int s = blockIdx.y;
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)inner * n_state) return;
  const int c = (int)(i / n_state);
  const int len = q_start[s + 1] - q_start[s];
  const int n_chunks = (len + chunk - 1) / chunk;
  const int slot = state_slots[s];
  const float A = a2[i];
  float S = slot >= 0 ? state[(size_t)slot * state_ld + i] : 0.f;
  for (int k0 = 0; k0 < n_chunks; k0 += 8) {         // eight chunks' numbers asked for at once, then walked in order
    float own[8], sdt[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int k = k0 + u < n_chunks ? k0 + u : n_chunks - 1;
      own[u] = chunk_state[((size_t)s * max_chunks + k) * inner * n_state + i];
      sdt[u] = chunk_dt[((size_t)s * max_chunks + k) * inner + c];
    }
    float start[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      start[u] = S;
      if (k0 + u < n_chunks) {
        const float e = A * sdt[u];
        S = (fast ? __builtin_amdgcn_exp2f(e) : expf(e)) * S + own[u];
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (k0 + u < n_chunks) chunk_state[((size_t)s * max_chunks + k0 + u) * inner * n_state + i] = start[u];
  }
  if (slot >= 0 && n_chunks > 0) state[(size_t)slot * state_ld + i] = S;
}

static int scan_lanes(int n_state) {
  int L = 1;
  while (L * SCAN_SPT < n_state) L *= 2;
  return L;
}

extern "C" int da_selective_scan(const void* x, int dtype, int x_ld, const float* raw, int raw_ld, const void* bc, int bc_ld,
                                 int b_off, int c_off, const void* z, int z_ld, const float* a2,
                                 const void* d, int d_dtype, float* state, long state_ld, const int* state_slots,
                                 const int* q_start, void* y, int y_ld, int S, int inner, int n_state, int chunk,
                                 int max_chunks, float* chunk_state, float* chunk_dt, void* stream) {
  DA_REQUIRE(S >= 0 && inner > 0 && n_state > 0 && x_ld >= inner && raw_ld >= inner && z_ld >= inner && y_ld >= inner,
             "selective_scan: bad sizes");
  DA_REQUIRE(b_off >= 0 && c_off >= 0 && b_off + n_state <= bc_ld && c_off + n_state <= bc_ld, "selective_scan: B or C leave the row");
  DA_REQUIRE(state_ld >= (long)inner * n_state, "selective_scan: the state row is too short");
  const int L = scan_lanes(n_state);
  DA_REQUIRE(L <= DA_WAVE, "selective_scan: %d state entries a channel, %d are taken", n_state, DA_WAVE * SCAN_SPT);
  DA_REQUIRE(chunk == 0 || (chunk > 0 && max_chunks > 0 && chunk_state && chunk_dt), "selective_scan: chunks need their workspace");
  if (S == 0) return 0;
  ScanIn in{x, x_ld, raw, raw_ld, bc, bc_ld, b_off, c_off, z, z_ld, a2, d, d_dtype};
  hipStream_t st = (hipStream_t)stream;
  const int gx = da_ceil_div((long)inner * L, SCAN_BLOCK);
#define DA_SCAN_GO(T)                                                                                                        \
  if (chunk == 0) {                                                                                                          \
    hipLaunchKernelGGL((selective_scan_kernel<T, 0>), dim3(gx, S), dim3(SCAN_BLOCK), 0, st, in, state, state_ld, state_slots, \
                       q_start, (T*)y, y_ld, inner, n_state, L, 0, nullptr, nullptr, 0);                                      \
  } else {                                                                                                                   \
    hipLaunchKernelGGL((selective_scan_kernel<T, 1>), dim3(gx, S, max_chunks), dim3(SCAN_BLOCK), 0, st, in, state, state_ld,  \
                       state_slots, q_start, (T*)y, y_ld, inner, n_state, L, chunk, chunk_state, chunk_dt, max_chunks);       \
    hipLaunchKernelGGL(scan_chunk_carry_kernel, dim3(da_ceil_div((long)inner * n_state, 256), S), dim3(256), 0, st,          \
                       chunk_state, chunk_dt, max_chunks, chunk, state, state_ld, state_slots, q_start, a2, inner, n_state, (int)(sizeof(T) == 2));  \
    hipLaunchKernelGGL((selective_scan_kernel<T, 2>), dim3(gx, S, max_chunks), dim3(SCAN_BLOCK), 0, st, in, state, state_ld,  \
                       state_slots, q_start, (T*)y, y_ld, inner, n_state, L, chunk, chunk_state, chunk_dt, max_chunks);       \
  }
  if (dtype == DA_BF16) { DA_SCAN_GO(bf16_t) } else { DA_SCAN_GO(float) }
#undef DA_SCAN_GO
  DA_CHECK_LAUNCH("selective_scan");
  return 0;
}
