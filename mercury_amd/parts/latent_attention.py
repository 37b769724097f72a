"""Causal softmax attention whose keys and values are functions of one cached latent."""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops
from .base import CacheSpec, Mixer, PositionEncoding, TensorSpec
from .lowering import OneOp

# Leaf names of the stored tensors, under the prefix the builder gives.
DEFAULT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv",
                 "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "q": "q",
                 "sink": "sink", "gate": "g"}


class LatentAttention(Mixer):
    """Attention through low-rank latents.

    With x the mixer's input [hidden], H heads of `dim` unrotated and `rot_dim` rotated
    query/key dims and `vdim` value dims:

        c_q = rmsnorm(W_dq x) * g_q                      (q_rank)
        q_h = (W_uq c_q)[h] = [q_h^n (dim) | q_h^r (rot_dim)]
        [c' | r'] = W_dkv x,  c = rmsnorm(c') * g_kv     (kv_rank), r = R_p r' (rot_dim)
        k_h^n = W_uk[h] c,  v_h = W_uv[h] c
        score_h(i, j) = scale * (q_h^n(i) . k_h^n(j) + R_i q_h^r(i) . r(j)),  j <= i
        out = W_o concat_h(sum_j softmax_j(score_h(i, .)) v_h(j))

    R_p turns the first `position.rotary_dim` dims of a rotated part by the position's angles.
    Only c and r are cached (one shared key/value head): the unrotated score is computed as
    (W_uk[h]^T q_h^n) . c and the head's output as W_uv[h] (sum_j p_j c_j), so neither keys nor
    values of the heads are ever expanded.  The cache holds a key row [c | r] per token and c
    once more, transposed within the page, as the value.  Norms, rotation, scores and softmax
    are float32 in either dtype.

    `q_rank` 0: there is no query latent; q = W_q x with ``<q>.weight`` [H (dim + rot_dim),
    hidden].  `window`: a query sees itself and the window - 1 tokens before it (the cache keeps
    no more).  `sinks`: a stored number per head (``<sink>.weight`` [H]) whose exponential
    stands once more in the softmax's denominator, unscaled, with no key or value behind it.
    `out_gate`: a projection ``<gate>.weight`` [H vdim, hidden] of the mixer's input whose
    sigmoid multiplies the heads' values side by side before the output projection.
    """

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int,
                 kv_rank: int, position: PositionEncoding, eps: float, scale: float | None = None,
                 window: int | None = None, names: dict | None = None, sinks: bool = False,
                 out_gate: bool = False):
        self.hidden, self.heads = int(hidden), int(heads)
        self.dim, self.rot_dim, self.vdim = int(dim), int(rot_dim), int(vdim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        if min(self.hidden, self.heads, self.dim, self.vdim, self.kv_rank) <= 0 \
                or self.rot_dim < 0 or self.q_rank < 0:
            raise ValueError("latent attention: sizes must be positive")
        self.position = position
        self.eps = float(eps)
        self.scale = float(scale) if scale is not None else (self.dim + self.rot_dim) ** -0.5
        self.window = int(window) if window else None
        self.sinks, self.out_gate = bool(sinks), bool(out_gate)
        self.sink = None
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_down = self.w_uq = self.w_uk_t = self.w_uv = self.w_o = None
        self.g_q = self.g_kv = None
        self._alone: dict = {}

    def cache_spec(self) -> CacheSpec:
        # one shared head; rows padded with zeros to a shape the matrix-core attention takes
        key_width, value_width = core.latent_cache_widths(self.kv_rank + self.rot_dim, self.kv_rank)
        return CacheSpec(1, key_width, self.window, value_dim=value_width)

    def param_specs(self) -> dict:
        n, per_head = self.names, self.dim + self.rot_dim
        if self.q_rank:
            specs = {
                f"{n['dq']}.weight": TensorSpec((self.q_rank, self.hidden)),
                f"{n['dq_norm']}.weight": TensorSpec((self.q_rank,), role="vector",
                                                     init="one_plus_normal"),
                f"{n['uq']}.weight": TensorSpec((self.heads * per_head, self.q_rank)),
            }
        else:
            specs = {f"{n['q']}.weight": TensorSpec((self.heads * per_head, self.hidden))}
        if self.sinks:
            specs[f"{n['sink']}.weight"] = TensorSpec((self.heads,), role="vector")
        if self.out_gate:
            specs[f"{n['gate']}.weight"] = TensorSpec((self.heads * self.vdim, self.hidden))
        return {
            **specs,
            f"{n['dkv']}.weight": TensorSpec((self.kv_rank + self.rot_dim, self.hidden)),
            f"{n['dkv_norm']}.weight": TensorSpec((self.kv_rank,), role="vector", init="one_plus_normal"),
            f"{n['uk']}.weight": TensorSpec((self.heads * self.dim, self.kv_rank)),
            f"{n['uv']}.weight": TensorSpec((self.heads * self.vdim, self.kv_rank)),
            f"{n['o']}.weight": TensorSpec((self.hidden, self.heads * self.vdim)),
        }

    def bind(self, params, dtype, device) -> None:
        n = self.names
        get = lambda key: params[f"{n[key]}.weight"]
        # one down-projection: rows [query latent | key/value latent | rotated key part | gate]
        down = ([get("dq")] if self.q_rank else []) + [get("dkv")] + \
               ([get("gate")] if self.out_gate else [])
        self.w_down = torch.cat(down, dim=0).contiguous()
        self.w_uq = get("uq") if self.q_rank else get("q")
        if self.sinks:
            self.sink = get("sink").float().contiguous()
        # W_uk of head h is [dim, kv_rank]; the absorbed query is W_uk[h]^T q, a product with
        # the transposed matrix as its [out, in] weight
        self.w_uk_t = get("uk").view(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = get("uv")
        self.w_o = get("o")
        norms = [get("dq_norm") if self.q_rank else get("dkv_norm"), get("dkv_norm")]
        common = torch.float32 if any(g.dtype == torch.float32 for g in norms) else dtype
        self.g_q, self.g_kv = (g.to(common).contiguous() for g in norms)
        if not self.q_rank:
            self.g_q = None
        self._alone.clear()

    def prepare(self, max_positions: int, device) -> None:
        self.position.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        tensors = (self.w_down, self.w_uq, self.w_uk_t, self.w_uv, self.w_o, self.g_q, self.g_kv,
                   self.sink)
        return sum(t.numel() * t.element_size() for t in tensors if t is not None)

    def lower(self, program, cache, state=None) -> None:
        pos = self.position.describe()
        if pos is None or pos.distance_slopes is not None:
            raise ValueError("latent attention takes a rotation by tabulated angles")
        if pos.rotary_dim > self.rot_dim:
            raise ValueError("more rotated dims than the rotated part holds")
        if cache.k.dtype != self.w_down.dtype:
            raise ValueError("the kernels keep the cached latents in the compute dtype")
        if not cache.writes:
            raise ValueError("latent attention writes its own cache")
        ptr = lambda t: 0 if t is None else t.data_ptr()
        program.append("latent_attention", core.latent_attention_params(
            w_down=self.w_down.data_ptr(), q_norm=ptr(self.g_q), kv_norm=self.g_kv.data_ptr(),
            norm_dtype=ops.dtype_code(self.g_kv.dtype), eps=self.eps, w_uq=self.w_uq.data_ptr(),
            w_uk_t=self.w_uk_t.data_ptr(), w_uv=self.w_uv.data_ptr(), w_o=self.w_o.data_ptr(),
            heads=self.heads, dim=self.dim, rot=self.rot_dim, vdim=self.vdim, q_rank=self.q_rank,
            kv_rank=self.kv_rank, rotary_dim=pos.rotary_dim, cos=ptr(pos.cos), sin=ptr(pos.sin),
            table_positions=0 if pos.cos is None else pos.cos.shape[0],
            interleaved=pos.interleaved, k_cache=cache.k.data_ptr(), v_cache=cache.v.data_ptr(),
            group=cache.group, page_size=cache.page_size, scale=self.scale,
            window=self.window or 0, writes=True, sinks=ptr(self.sink), out_gate=self.out_gate))

    def forward(self, x, step, cache, state, accum):
        # the operation `lower` appends, as a program of its own
        key = (cache.k.data_ptr(), cache.group)
        alone = self._alone.get(key)
        if alone is None:
            alone = self._alone[key] = OneOp(x.dtype, self.hidden, 0,
                                             lambda program: self.lower(program, cache))
        _logits, _x, pending = alone.run(step, accum, x=x)
        return pending
