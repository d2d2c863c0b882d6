"""Mixers that carry a matrix of state a head from token to token instead of keys."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.pages import StateSpec
from ..errors import Unsupported
from ..kernels import ops
from .base import StepContext, settled
from .linear import linear
from .norms import as_tensor
from .registry import register_mixer


class WKV:
    """Five mixes of a token's input with the one before it, m_c = h + (h_prev - h) * mu_c, feed receptance, key, value, gate
    and a low-rank decay w = exp(-exp(W2 tanh(W1 m_w) + w0)); per head o = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T;
    o is brought to unit root mean square over the head, times a weight and silu(gate), then the output projection. A request's
    slot holds the heads' matrices and the last row of h, all 32-bit; the products' results stay 32-bit up to the recurrence."""

    replayable = True
    takes_padding_rows = True  # (the recurrence walks the requests' own rows; rows behind them are computed by the products only)

    MIXES = ("r", "k", "v", "g", "w")
    GROUPED_ROWS = 128  # steps of up to this many rows run the four products as one grouped launch

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.n_head, self.head_dim, self.rank, self.eps = spec.width, spec.n_head, spec.head_dim, spec.decay_rank, float(spec.eps)
        H, D, d, R = self.n_head, self.head_dim, self.width, self.rank
        if not ops.scan_takes(D, D):
            raise Unsupported(f"wkv: heads of {D} are not supported")
        t = spec.tensors
        self.mu = store.fetch_joined([t["mu_" + c] for c in self.MIXES], [(d,)] * 5, "vector", "stack")
        # receptance, key, value and gate: one matrix a mix, stacked, so that steps of few rows run them as one launch
        self.weights = store.fetch_joined([t[c] for c in ("r", "k", "v", "g")], [(H * D, d)] * 4, "matrix", "stack")
        self.w1 = store.fetch(t["w1"], (R, d), "matrix")
        self.w2 = store.fetch(t["w2"], (H * D, R), "matrix")
        self.w0 = store.fetch(t["w0"], (H * D,), "vector")
        self.u = store.fetch(t["u"], (H, D), "vector").reshape(H * D)
        self.norm = store.fetch(t["norm"], (H * D,), "vector")
        self.out_weight = store.fetch(t["out"], (d, H * D), "matrix")

    def cache_spec(self):
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.n_head * self.head_dim * self.head_dim + self.width,))

    def forward(self, h, ctx: StepContext, cache, state, residual: Optional[torch.Tensor], writes_cache: bool = True,
                out: Optional[torch.Tensor] = None):
        h = as_tensor(h)
        n, ws, HD = h.shape[0], ctx.workspace, self.n_head * self.head_dim
        d = self.width
        mixes = ws.get("wkv_mixes", (n, 5, d), self.dtype)
        ops.token_shift(mixes, h, self.mu, state, HD * self.head_dim, ctx)
        mixes = mixes.view(n, 5 * d)
        proj = ws.get("wkv_proj", (n, 5 * HD), torch.float32)
        if n <= self.GROUPED_ROWS:
            # four products of four inputs in one launch (a step of few rows is a chain of launches, not of bytes)
            ops.heads_product(proj[:, :4 * HD], mixes[:, :4 * d], self.weights)
        else:
            for c in range(4):
                linear(mixes[:, c * d:(c + 1) * d], self.weights[c], None, out=proj[:, c * HD:(c + 1) * HD])
        low = ws.get("wkv_low", (n, self.rank), torch.float32)
        linear(mixes[:, 4 * d:], self.w1, None, out=low)
        low_act = ws.get("wkv_low_act", (n, self.rank), self.dtype)
        ops.activate(low_act, low, "tanh")
        linear(low_act, self.w2, None, out=proj[:, 4 * HD:])
        y = ws.get("wkv_out", (n, HD), self.dtype)
        ops.wkv_scan(y, proj, self.w0, self.u, self.norm, self.eps, state, h, ctx, n_head=self.n_head, head_dim=self.head_dim)
        if out is not None:
            linear(y, self.out_weight, None, out=out)
        else:
            linear(y, self.out_weight, None, residual=settled(residual))
        return None


class StateSpace:
    """[z | x | B | C | dt] = Win h (kept 32-bit); (x, B, C) <- silu(conv(.) + bias) over the request's own rows in time; dt <-
    softplus(dt + dt_bias); per head S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x, heads sharing B and C in groups;
    y * silu(z), unit root mean square in `norm_groups` parts, a weight, the output projection. A request's slot holds the
    heads' matrices [heads, state, head_dim] and the last taps - 1 rows of (x, B, C) before the convolution, all 32-bit."""

    replayable = True
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.n_head, self.head_dim = spec.width, spec.n_head, spec.head_dim
        self.n_state, self.n_groups, self.taps, self.norm_groups, self.eps = spec.n_state, spec.n_groups, int(spec.taps), spec.norm_groups, float(spec.eps)
        H, P, N, G, d = self.n_head, self.head_dim, self.n_state, self.n_groups, self.width
        self.inner = H * P
        self.channels = self.inner + 2 * G * N
        if H % G or self.inner % self.norm_groups or self.taps < 1:
            raise ValueError(f"state space: {H} heads in {G} groups, {self.inner} channels in {self.norm_groups} norm parts, {self.taps} taps")
        if not ops.scan_takes(N, P):
            raise Unsupported(f"state space: a state of {N} x {P} a head is not supported")
        t = spec.tensors
        self.in_weight = store.fetch(t["in"], (2 * self.inner + 2 * G * N + H, d), "matrix")
        self.conv = store.fetch(t["conv"], (self.channels, self.taps), "vector")
        self.conv_bias = store.fetch(t["conv_bias"], (self.channels,), "vector") if "conv_bias" in t else None
        self.dt_bias = store.fetch(t["dt_bias"], (H,), "vector")
        self.a_log = store.fetch(t["A_log"], (H,), "vector")
        self.d_skip = store.fetch(t["D"], (H,), "vector")
        self.norm = store.fetch(t["norm"], (self.inner,), "vector")
        self.out_weight = store.fetch(t["out"], (d, self.inner), "matrix")

    def cache_spec(self):
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.inner * self.n_state + (self.taps - 1) * self.channels,))

    def forward(self, h, ctx: StepContext, cache, state, residual: Optional[torch.Tensor], writes_cache: bool = True,
                out: Optional[torch.Tensor] = None, proj: Optional[torch.Tensor] = None):
        """`proj`: the input projection's 32-bit rows, when the caller has made them (as columns of a wider product)."""
        n, ws, inner, C = h.shape[0], ctx.workspace, self.inner, self.channels
        if proj is None:
            proj = ws.get("ssm_in", (n, self.in_weight.shape[0]), torch.float32)
            linear(h, self.in_weight, None, out=proj)
        raw = proj[:, inner:inner + C]
        xbc = ws.get("ssm_xbc", (n, C), torch.float32)
        ops.conv_act(xbc, raw, self.conv, self.conv_bias, state, inner * self.n_state, ctx)
        y = ws.get("ssm_y", (n, inner), torch.float32)
        ops.ssd_scan(y, xbc, proj[:, inner + C:], self.dt_bias, self.a_log, self.d_skip, state, raw if self.taps > 1 else None,
                     self.taps - 1, ctx, n_head=self.n_head, head_dim=self.head_dim, n_state=self.n_state, n_groups=self.n_groups)
        normed = ws.get("ssm_normed", (n, inner), self.dtype)
        ops.gated_group_norm(normed, y, proj[:, :inner], self.norm, self.eps, self.norm_groups)
        if out is not None:
            linear(normed, self.out_weight, None, out=out)
        else:
            linear(normed, self.out_weight, None, residual=settled(residual))
        return None


register_mixer("wkv", WKV)
register_mixer("state_space", StateSpace)
