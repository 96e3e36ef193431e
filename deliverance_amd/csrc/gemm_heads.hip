// A product per head on the matrix cores (bfloat16): out[:, h, :n] = a[:, h, :k] @ w[h].T for a stack w [H][n][k],
// the heads' pieces lying side by side in the rows of a and of out (a_hs, o_hs entries apart, from a_off, o_off on).
// Latent attention folds every head's key map into its query with it, and applies every head's value map to the
// head's weighted sum.  A workgroup of four wavefronts owns 32 rows x 64 columns of one head (MFMA 16x16x32,
// operands from memory straight into the lanes' fragments, four k-steps asked for at once); a row's sums run over
// k in ascending order whatever else is in the step.
#include "gemm_common.h"

#define GH_ROWS 32
#define GH_COLS 64
#define GH_UNROLL 4

__global__ void __launch_bounds__(256)
gemm_heads_kernel(const bf16_t* __restrict__ a, int lda, int a_hs, int a_off, const bf16_t* __restrict__ w,
                  bf16_t* __restrict__ out, int ldo, int o_hs, int o_off, int M, int n, int k) {
  const int h = blockIdx.z;
  const int t = threadIdx.x, lane = t % DA_WAVE, wave = t / DA_WAVE;
  const int fr = lane % 16, fk = (lane / 16) * 8;
  const int m0 = blockIdx.y * GH_ROWS, n0 = blockIdx.x * GH_COLS + wave * 16;
  if (n0 >= n) return;
  const bf16_t* ap[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = m0 + i * 16 + fr;
    ap[i] = a + (size_t)(r < M ? r : M - 1) * lda + (size_t)h * a_hs + a_off + fk;     // rows past the end are never stored
  }
  const int wcol = n0 + fr < n ? n0 + fr : 0;
  const bf16_t* wp = w + ((size_t)h * n + wcol) * k + fk;
  floatx4 acc[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int k0 = 0; k0 < k; k0 += 32 * GH_UNROLL) {
    uint4 av[GH_UNROLL][2], wv[GH_UNROLL];
#pragma unroll
    for (int u = 0; u < GH_UNROLL; ++u) {
      const int kk = k0 + u * 32;
      const int ks = (kk + fk < k) ? kk : -fk;          // past k: the row's first piece, met by zeros in a
      av[u][0] = load16(ap[0] + ks);
      av[u][1] = load16(ap[1] + ks);
      wv[u] = load16(wp + ks);
    }
#pragma unroll
    for (int u = 0; u < GH_UNROLL; ++u) {
      const bool kin = k0 + u * 32 + fk < k;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint4 x = kin ? av[u][i] : zero;
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, x), __builtin_bit_cast(bf16x8_t, wv[u]),
                                                         acc[i], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = m0 + i * 16 + 4 * (lane / 16) + r;
      if (row >= M || n0 + fr >= n) continue;
      out[(size_t)row * ldo + (size_t)h * o_hs + o_off + n0 + fr] = f32_to_bf16(acc[i][r]);
    }
}

extern "C" int da_gemm_heads_takes(int lda, int a_hs, int a_off, int k) {
  return k % 8 == 0 && lda % 8 == 0 && a_hs % 8 == 0 && a_off % 8 == 0;
}

extern "C" int da_gemm_heads(const void* a, int lda, int a_hs, int a_off, const void* w, void* out, int ldo, int o_hs,
                             int o_off, int M, int H, int n, int k, void* stream) {
  DA_REQUIRE(M >= 0 && H > 0 && n > 0 && k > 0 && a_off >= 0 && o_off >= 0, "gemm_heads: bad sizes");
  DA_REQUIRE(da_gemm_heads_takes(lda, a_hs, a_off, k) && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0,
             "gemm_heads: k, the row length of a and the heads' places must be multiples of 8, operands 16-byte aligned");
  DA_REQUIRE(lda >= (long)(H - 1) * a_hs + a_off + k && ldo >= (long)(H - 1) * o_hs + o_off + n, "gemm_heads: the heads leave the rows");
  if (M == 0) return 0;
  hipLaunchKernelGGL(gemm_heads_kernel, dim3(da_ceil_div(n, GH_COLS), da_ceil_div(M, GH_ROWS), H), dim3(256), 0,
                     (hipStream_t)stream, (const bf16_t*)a, lda, a_hs, a_off, (const bf16_t*)w, (bf16_t*)out, ldo, o_hs, o_off,
                     M, n, k);
  DA_CHECK_LAUNCH("gemm_heads");
  return 0;
}
