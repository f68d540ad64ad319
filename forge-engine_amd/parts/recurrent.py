"""Mixers that carry a matrix state per head from token to token instead of a cache of keys.

All three are the linear recurrence

    S_t = diag(a_t) S_(t-1) + b_t k_t v_t^T            (S: [key dim, value dim] per head, float32)

read by a query, and differ in where the decay a_t and the input scale b_t come from, whether the
query reads the state before or after the token's own update, and how the read-out is
normalised.  One kernel runs the recurrence for all of them (``ops.linear_recurrence``), for
prompt portions and single tokens alike; the state of every live request lives in a fixed-size
slot, so a request may be cut into steps anywhere.  Decays, gates, the state and the read-out
are float32 in both compute modes; the projections run in the compute dtype.

* ``rwkv_time_mix``: every projection reads its own blend of the token's input and the previous
  token's, ``x_t + (x_(t-1) - x_t) * mu_s``; decay per key channel ``exp(-exp(W2 tanh(W1 x_w) + w0))``;
  the query (receptance) reads ``S_(t-1) + diag(u) k_t v_t^T``, the bonus u counting for the
  current token only; heads normalised to unit root mean square, times a weight, times silu(gate).
* ``gated_linear_attention``: decay per key channel ``sigmoid(W2 (W1 x) + b)^(1/tau)``; the query,
  scaled by dim^-1/2, reads S_t; heads RMS-normed with one weight of the value size shared by all
  heads, times silu(gate).
* ``mlstm``: one log input gate and one log forget gate per head, both bounded by
  ``cap * tanh(. / cap)``, the forget gate then through logsigmoid; a running maximum m (from 0)
  keeps the exponentials in range: ``m_t = max(f + m_(t-1), i)``, a_t = exp(f + m_(t-1) - m_t),
  b_t = exp(i - m_t); a normaliser n_t follows the same recurrence with k alone (kept as one more
  column of the state, fed by v = 1); read-out ``S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)``,
  heads normalised to unit root mean square, times a weight, times sigmoid(gate).
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView, FixedState
from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Mixer, ParamSpec


class _RecurrentMixer(Mixer):
    """Shared plumbing: a table of checkpoint names, matrices that read the same input fused
    into one product."""

    DEFAULT_NAMES: dict[str, str] = {}
    STATE = "matrix"

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, heads: int, key_dim: int,
                 value_dim: int, eps: float, names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size, self.heads, self.key_dim, self.value_dim = hidden_size, heads, key_dim, value_dim
        self.eps = float(eps)
        self.names = dict(self.DEFAULT_NAMES, **(names or {}))
        self.tensors: dict[str, Tensor] = {}
        self._fused: dict[str, tuple[str, int, int]] = {}     # key -> (fused name, first row, rows)
        self._fused_rows: dict[str, int] = {}

    def fuse(self, fused: str, keys_and_rows: list[tuple[str, int]]) -> None:
        at = 0
        for key, rows in keys_and_rows:
            self._fused[key] = (fused, at, rows)
            at += rows
        self._fused_rows[fused] = at

    def shapes(self) -> dict[str, tuple[tuple[int, ...], str, str]]:
        """key -> (shape, kind, init) of every tensor."""
        raise NotImplementedError

    def param_specs(self):
        return {self.name(self.names[key]): ParamSpec(shape, kind=kind, init=init)
                for key, (shape, kind, init) in self.shapes().items()}

    def set_param(self, name: str, tensor: Tensor) -> None:
        local = name[len(self.prefix) + 1:] if self.prefix else name
        key = next((k for k, leaf in self.names.items() if leaf == local and k in self.shapes()), None)
        if key is None:
            raise KeyError(name)
        if key in self._fused:
            fused, at, rows = self._fused[key]
            if fused not in self.tensors:
                self.tensors[fused] = torch.empty((self._fused_rows[fused], tensor.shape[1]), dtype=tensor.dtype,
                                                  device=tensor.device)
            if tensor.dtype != self.tensors[fused].dtype:
                raise ValueError(f"{name}: the projections of one input must be stored in one dtype")
            self.tensors[fused][at:at + rows].copy_(tensor)
        else:
            self.tensors[key] = tensor

    def columns(self, product: Tensor, key: str) -> Tensor:
        """The columns of a fused product that belong to one projection (a strided view)."""
        _, at, rows = self._fused[key]
        return product[:, at:at + rows]

    def state_shape(self) -> tuple[int, ...]:
        return (self.heads, self.value_dim, self.key_dim)      # value-major: a thread's key channels lie together

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(state={self.STATE: FixedState(self.state_shape(), torch.float32)})

    def kernel_libraries(self):
        return {"linear_recurrence", "stream_ops", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


class RWKVTimeMix(_RecurrentMixer):
    DEFAULT_NAMES = {"mu_r": "mu.r", "mu_k": "mu.k", "mu_v": "mu.v", "mu_g": "mu.g", "mu_w": "mu.w",
                     "r": "r", "k": "k", "v": "v", "g": "g", "w1": "w1", "w2": "w2", "w0": "w0", "u": "u",
                     "norm": "norm", "o": "o"}
    PREVIOUS = "previous"
    MIXES = ("mu_r", "mu_k", "mu_v", "mu_g", "mu_w")

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, heads: int, dim: int, eps: float,
                 decay_rank: int, names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix, hidden_size=hidden_size, heads=heads, key_dim=dim, value_dim=dim, eps=eps,
                         names=names)
        self.decay_rank = decay_rank
        self.mu: Tensor | None = None

    def shapes(self):
        size, width = self.heads * self.key_dim, self.hidden_size
        found = {key: ((width,), "vector", "uniform") for key in self.MIXES}
        found.update({key: ((size, width), "matrix", "normal") for key in ("r", "k", "v", "g")})
        found.update(w1=((self.decay_rank, width), "matrix", "normal"), w2=((size, self.decay_rank), "matrix", "normal"),
                     w0=((size,), "vector", "unit"), u=((self.heads, self.key_dim), "vector", "unit"),
                     norm=((size,), "vector", "norm"), o=((width, size), "matrix", "normal"))
        return found

    def set_param(self, name: str, tensor: Tensor) -> None:
        super().set_param(name, tensor)
        for index, key in enumerate(self.MIXES):
            if key in self.tensors:
                if self.mu is None:
                    self.mu = torch.zeros((len(self.MIXES), self.hidden_size), dtype=torch.float32, device=tensor.device)
                self.mu[index].copy_(self.tensors.pop(key))

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(state={self.STATE: FixedState(self.state_shape(), torch.float32),
                                 self.PREVIOUS: FixedState((self.hidden_size,), torch.float32)})

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True) -> Tensor:
        t = self.tensors
        mixes = ops.token_shift(x, self.mu, cache.states[self.PREVIOUS], batch.cu_q, batch.token_seq,
                                batch.state_slots, num_seqs=batch.num_seqs, out_dtype=x.dtype)
        r = ops.linear(mixes[0], t["r"])
        k = ops.linear(mixes[1], t["k"])
        v = ops.linear(mixes[2], t["v"])
        gate = ops.linear(mixes[3], t["g"])
        low = ops.tanh_rows(ops.linear(mixes[4], t["w1"]))
        decay = ops.linear(low, t["w2"], out_dtype=torch.float32)
        out = torch.empty((x.shape[0], self.heads, self.value_dim), dtype=torch.float32, device=x.device)
        ops.linear_recurrence(r, k, v, out, cache.states[self.STATE], batch.cu_q, batch.state_slots,
                              num_seqs=batch.num_seqs, max_q_len=batch.max_q_len, heads=self.heads,
                              key_dim=self.key_dim, value_dim=self.value_dim, decay=decay,
                              decay_kind="exp_neg_exp", decay_bias=t["w0"], bonus=t["u"])
        y = torch.empty((x.shape[0], self.heads * self.value_dim), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(out, t["norm"], gate, y, heads=self.heads, dim=self.value_dim, eps=self.eps, act="silu")
        return ops.linear_update(y, t["o"])


class GatedLinearAttention(_RecurrentMixer):
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2",
                     "a2_bias": "a2.b"}

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, heads: int, dim: int, value_dim: int,
                 eps: float, tau: float, decay_rank: int, names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix, hidden_size=hidden_size, heads=heads, key_dim=dim, value_dim=value_dim, eps=eps,
                         names=names)
        self.tau = float(tau)
        self.decay_rank = decay_rank
        self.fuse("qkvg", [("q", heads * dim), ("k", heads * dim), ("v", heads * value_dim), ("g", heads * value_dim)])

    def shapes(self):
        keys, values, width = self.heads * self.key_dim, self.heads * self.value_dim, self.hidden_size
        return {"q": ((keys, width), "matrix", "normal"), "k": ((keys, width), "matrix", "normal"),
                "v": ((values, width), "matrix", "normal"), "g": ((values, width), "matrix", "normal"),
                "o": ((width, values), "matrix", "normal"), "norm": ((self.value_dim,), "vector", "norm"),
                "a1": ((self.decay_rank, width), "matrix", "normal"), "a2": ((keys, self.decay_rank), "matrix", "normal"),
                "a2_bias": ((keys,), "vector", "unit")}

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True) -> Tensor:
        t = self.tensors
        qkvg = ops.linear(x, t["qkvg"])
        decay = ops.linear(ops.linear(x, t["a1"]), t["a2"], out_dtype=torch.float32)
        out = torch.empty((x.shape[0], self.heads, self.value_dim), dtype=torch.float32, device=x.device)
        ops.linear_recurrence(self.columns(qkvg, "q"), self.columns(qkvg, "k"), self.columns(qkvg, "v"), out,
                              cache.states[self.STATE], batch.cu_q, batch.state_slots, num_seqs=batch.num_seqs,
                              max_q_len=batch.max_q_len, heads=self.heads, key_dim=self.key_dim,
                              value_dim=self.value_dim, decay=decay, decay_kind="sigmoid_root",
                              decay_bias=t["a2_bias"], tau=self.tau, q_scale=self.key_dim ** -0.5)
        y = torch.empty((x.shape[0], self.heads * self.value_dim), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(out, t["norm"], self.columns(qkvg, "g"), y, heads=self.heads, dim=self.value_dim,
                           eps=self.eps, act="silu")
        return ops.linear_update(y, t["o"])


class MLSTM(_RecurrentMixer):
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "f": "f",
                     "i_bias": "i.b", "f_bias": "f.b"}
    MAXIMUM = "maximum"

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, heads: int, dim: int, value_dim: int,
                 eps: float, gate_cap: float, names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix, hidden_size=hidden_size, heads=heads, key_dim=dim, value_dim=value_dim, eps=eps,
                         names=names)
        self.gate_cap = float(gate_cap)
        self.fuse("qkvg", [("q", heads * dim), ("k", heads * dim), ("v", heads * value_dim), ("g", heads * value_dim)])
        self.fuse("gates", [("i", heads), ("f", heads)])
        self.gate_bias: Tensor | None = None

    def shapes(self):
        keys, values, width = self.heads * self.key_dim, self.heads * self.value_dim, self.hidden_size
        return {"q": ((keys, width), "matrix", "normal"), "k": ((keys, width), "matrix", "normal"),
                "v": ((values, width), "matrix", "normal"), "g": ((values, width), "matrix", "normal"),
                "o": ((width, values), "matrix", "normal"), "norm": ((values,), "vector", "norm"),
                "i": ((self.heads, width), "matrix", "normal"), "f": ((self.heads, width), "matrix", "normal"),
                "i_bias": ((self.heads,), "vector", "unit"), "f_bias": ((self.heads,), "vector", "unit")}

    def set_param(self, name: str, tensor: Tensor) -> None:
        super().set_param(name, tensor)
        for index, key in enumerate(("i_bias", "f_bias")):
            if key in self.tensors:
                if self.gate_bias is None:
                    self.gate_bias = torch.zeros(2 * self.heads, dtype=torch.float32, device=tensor.device)
                self.gate_bias[index * self.heads:(index + 1) * self.heads].copy_(self.tensors.pop(key))

    def state_shape(self) -> tuple[int, ...]:
        return (self.heads, self.value_dim + 1, self.key_dim)     # the normaliser is one more value column

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(state={self.STATE: FixedState(self.state_shape(), torch.float32),
                                 self.MAXIMUM: FixedState((self.heads,), torch.float32)})

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True) -> Tensor:
        t = self.tensors
        qkvg = ops.linear(x, t["qkvg"])
        gates = ops.linear(x, t["gates"], out_dtype=torch.float32)
        scanned = torch.empty((3, x.shape[0], self.heads), dtype=torch.float32, device=x.device)
        ops.mlstm_gate_scan(gates, self.gate_bias, self.gate_cap, cache.states[self.MAXIMUM], batch.cu_q,
                            batch.state_slots, scanned, num_seqs=batch.num_seqs, heads=self.heads)
        out = torch.empty((x.shape[0], self.heads, self.value_dim + 1), dtype=torch.float32, device=x.device)
        ops.linear_recurrence(self.columns(qkvg, "q"), self.columns(qkvg, "k"), self.columns(qkvg, "v"), out,
                              cache.states[self.STATE], batch.cu_q, batch.state_slots, num_seqs=batch.num_seqs,
                              max_q_len=batch.max_q_len, heads=self.heads, key_dim=self.key_dim,
                              value_dim=self.value_dim, head_decay=scanned[0], in_scale=scanned[1],
                              q_scale=self.key_dim ** -0.5, ones_column=True)
        y = torch.empty((x.shape[0], self.heads * self.value_dim), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(out, t["norm"], self.columns(qkvg, "g"), y, heads=self.heads, dim=self.value_dim,
                           eps=self.eps, act="sigmoid", extra=1, floor=scanned[2])
        return ops.linear_update(y, t["o"])


register_part("mixer", "rwkv_time_mix", RWKVTimeMix)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "mlstm", MLSTM)
