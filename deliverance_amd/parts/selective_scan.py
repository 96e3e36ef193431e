"""A selective state-space mixer (``SelectiveScanSpec``): up-projection to [x | z], a short causal filter and SiLU
on x, step sizes and the vectors B and C from x, the scan, the gate silu(z), and the down-projection added into
the stream.  A request's state is one 32-bit row [ S: inner x state | the filter's last taps - 1 inputs ]; the
kernels find each sequence's row through ``ctx.state_slots`` on the device, so decode steps can be recorded.
What enters the recurrence (step sizes before and after softplus, decays, the state, the gate) is 32-bit."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Mixer, StateNeed, StepContext, register_mixer, to_matrix, to_vector


class SelectiveScan(Mixer):
    graph_safe = True
    can_store = True

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        E, I, n, r, K = spec.width, spec.inner, spec.state, spec.dt_rank, spec.conv_taps
        self.inner, self.state, self.dt_rank, self.taps = I, n, r, K
        if not (1 <= K <= ops.CONV_MAX_TAPS):
            raise ValueError(f"a filter of {K} taps is outside 1..{ops.CONV_MAX_TAPS}")
        if not (1 <= n <= ops.SCAN_MAX_STATE):
            raise ValueError(f"{n} state entries a channel are outside 1..{ops.SCAN_MAX_STATE}")

        def shaped(name, shape):
            t = params[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name} is {list(t.shape)}, expected {list(shape)}")
            return t

        self.in_weight = to_matrix(shaped("in_weight", (2 * I, E)), dtype, device)
        self.conv_weight = to_vector(shaped("conv_weight", (I, K)), dtype, device)
        self.conv_bias = to_vector(shaped("conv_bias", (I,)), dtype, device)
        self.x_weight = to_matrix(shaped("x_weight", (r + 2 * n, I)), dtype, device)
        self.dt_weight = to_matrix(shaped("dt_weight", (I, r)), dtype, device)
        self.dt_bias = to_vector(shaped("dt_bias", (I,)), dtype, device)
        # A = -exp(A_log) in 32-bit (times log2(e) for bfloat16 rows: what the scan kernel takes)
        self.rates = ops.scan_rates(shaped("a_log", (I, n)).to(device), dtype)
        self.d = to_vector(shaped("d", (I,)), dtype, device)
        self.out_weight = to_matrix(shaped("out_weight", (E, I)), dtype, device)
        self.conv_off = I * n                      # where the filter's inputs start in a state row

    def cache_need(self):
        return StateNeed(self.inner * self.state + (self.taps - 1) * self.inner)

    normed_into = True

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor, call, into=None) -> bool:
        """Small steps: the root-mean-square norm in front and the up-projection in one kernel."""
        N = x.shape[0]
        rms = getattr(norm, "rms_params", lambda: None)()
        if rms is None or not ops.can_fuse_ln(N, x, self.in_weight):
            return False
        gain, offset, eps = rms
        xz = ctx.buf("scan_xz", N, 2 * self.inner, ctx.dtype)
        ops.linear_rms(x, None, N, gain, offset, eps, self.in_weight, None, xz)
        self._scan(ctx, xz, x if into is None else into, call)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        xz = ctx.buf("scan_xz", h.shape[0], 2 * self.inner, ctx.dtype)
        ops.linear(h, self.in_weight, None, xz)
        self._scan(ctx, xz, x, call)

    def _scan(self, ctx: StepContext, xz: torch.Tensor, x: torch.Tensor, call) -> None:
        N, I, n, r = xz.shape[0], self.inner, self.state, self.dt_rank
        state = ctx.cache.state[call.cache]                          # [slots, inner * state + (taps - 1) * inner]
        xc = ctx.buf("scan_x", N, I, ctx.dtype)
        ops.conv_causal(ctx, xz[:, :I], state, self.conv_off, self.conv_weight, self.conv_bias, "silu", xc)
        if call.write:
            ops.conv_state_update(ctx, xz[:, :I], state, self.conv_off, I, self.taps)
        proj = ctx.buf("scan_proj", N, r + 2 * n, ctx.dtype)
        ops.linear(xc, self.x_weight, None, proj)
        raw = ctx.buf("scan_dt", N, I, torch.float32)                # step sizes before softplus, unrounded
        ops.linear(proj[:, :r], self.dt_weight, self.dt_bias, raw)
        y = ctx.buf("scan_y", N, I, ctx.dtype)
        ops.selective_scan(ctx, xc, raw, proj, r, r + n, xz[:, I:], self.rates, self.d, state, y, n)
        ops.linear(y, self.out_weight, None, x, accumulate=ctx.part_accumulate)


register_mixer("selective_scan", SelectiveScan)
