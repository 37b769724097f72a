"""Causal grouped-query softmax attention over a paged cache."""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops
from .base import CacheSpec, Mixer, PositionEncoding, TensorSpec
from .lowering import OneOp

# Leaf names of the stored tensors, under the prefix the builder gives; an architecture whose
# checkpoints call them otherwise passes its own map.
DEFAULT_NAMES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj",
                 "q_norm": "q_norm", "k_norm": "k_norm", "sink": "sink", "gate": "g_proj",
                 "lq1": "lambda_q1", "lk1": "lambda_k1", "lq2": "lambda_q2", "lk2": "lambda_k2",
                 "v_mix": "v_mix"}
# the kernels' codes of `v_mix`
V_MIX_CODES = {None: 0, "leave": 1, "blend": 2}


class Attention(Mixer):
    """q/k/v projections (optionally biased), position encoding on q and k, keys and values
    written to the paged cache, softmax(q k^T * scale) v over the sequence's cached keys,
    output projection (optionally biased) added into the accumulator.

    Query head h reads key/value head h // (n_q / n_kv).  A query at absolute position p sees
    keys j <= p, and with a window only j > p - window
    (reference: mercury/model/qwen2.py:45-69, mercury/model/attention.py:9-32, :87-101).
    `names` maps q, k, v, o to the stored tensors' leaf names (default ``q_proj`` ...).
    `score_cap` bounds the scaled score to cap * tanh(score / cap); a position encoding may
    bring a penalty on the distance in the score (`PositionDescriptor.distance_slopes`).  The
    reference has neither; with either the float32-arithmetic attention kernel runs.

    Further makes of the same mixer, each a parameter:
    `values="keys"`: there is no v projection; the values are the keys as projected (with their
    bias), before any norm or rotation.  `value_dim`: values of another width than the keys.
    `qk_norm` ("whole"): an RMS norm over the whole q projection and one over the whole k
    projection (all heads at once; plain weights ``<q_norm>.weight`` [n_q d] and
    ``<k_norm>.weight`` [n_kv d], eps `norm_eps`), before the rotation; ("head"): the norm runs
    over every head by itself, with one weight of d entries for the query heads and one for the
    key heads.
    `q_temp=(coef, every)`: the query at position p is multiplied by
    1 + coef * ln(floor((p + 1) / every) + 1), after its norm.
    `sinks`: a stored number per query head (``<sink>.weight`` [n_q]) whose exponential stands
    once more in the softmax's denominator, unscaled, with no key or value behind it.
    `k_bias` / `v_bias` (default: as `qkv_bias`) say which of the projections have a bias.
    `keep_first` (with a `window`): the sequence's first `keep_first` keys stay visible to
    queries whose window has passed them, at their true positions.  `cache_window` /
    `cache_keep_first` widen what the cache keeps beyond this layer's own mask, for a slot that
    layers with other masks read.
    `maps=2`: differential attention.  `head_dim` is a head's whole key row, two score maps of
    head_dim / 2 dims side by side in the q and k projections (each map turned by itself over
    its first dims; `position` is built for a map's width); both maps are softmax attentions
    over the same values, combined as  o = a1 - lam * a2,
    lam = exp(<lq1, lk1>) - exp(<lq2, lk2>) + `diff_init`  (four stored vectors of a map's
    width, one number for the layer), then o / rms(o) over the head (eps `norm_eps`, no weight)
    times 1 - `diff_init`.  `head_gate`: a projection ``<gate>.weight`` [n_q, hidden] of the
    mixer's input gives one number a head, whose sigmoid multiplies the head's output before
    the output projection.
    `own_kv=False`: the layer has no key and value projections; it reads a cache slot that
    another layer writes (whose head counts, widths and rotation are its own).
    `out_gate`: a projection ``<gate>.weight`` [n_q value_dim, hidden] of the mixer's input whose
    sigmoid multiplies the heads' outputs side by side, column by column, before the output
    projection.
    `v_mix`: values mixed across layers.  ``"leave"``: the layer's values of a step's tokens, as
    projected, stay at hand for the layers after it; ``"blend"``: the layer caches and attends
    over (1 - lam) v + lam v_left, v_left being what a "leave" layer earlier in the execution
    list left for the same token and lam the stored number ``<v_mix>`` (a "leave" layer stores
    one too and does not use it; `v_mix_stored` says whether a layer that does not mix stores
    the number all the same: "yes", "maybe", "no").  Both kinds of layer have n_kv value_dim
    value columns alike.
    """

    graph_safe = True   # forward launches kernels only: a decode step may be captured in a graph

    def __init__(self, hidden: int, n_q: int, n_kv: int, head_dim: int,
                 position: PositionEncoding, qkv_bias: bool = True, o_bias: bool = False,
                 scale: float | None = None, window: int | None = None,
                 names: dict | None = None, score_cap: float | None = None,
                 values: str = "projected", value_dim: int | None = None,
                 qk_norm: str | None = None, norm_eps: float = 1e-6,
                 q_temp: tuple | None = None, sinks: bool = False, keep_first: int = 0,
                 maps: int = 1, diff_init: float = 0.0, head_gate: bool = False,
                 cache_window: int | None = -1, cache_keep_first: int | None = None,
                 own_kv: bool = True, out_gate: bool = False, v_mix: str | None = None,
                 v_mix_stored: str | None = None):
        if n_q % n_kv:
            raise ValueError(f"{n_q} query heads are not a multiple of {n_kv} key/value heads")
        self.hidden, self.n_q, self.n_kv, self.head_dim = int(hidden), int(n_q), int(n_kv), int(head_dim)
        self.position = position
        self.qkv_bias, self.o_bias = bool(qkv_bias), bool(o_bias)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.window = int(window) if window else None
        self.score_cap = float(score_cap) if score_cap else 0.0
        if values not in ("projected", "keys"):
            raise ValueError(f"values {values!r}: 'projected' or 'keys'")
        self.values_are_keys = values == "keys"
        self.value_dim = int(value_dim) if value_dim else self.head_dim
        if self.values_are_keys and self.value_dim != self.head_dim:
            raise ValueError("values that are the keys are as wide as the keys")
        if qk_norm not in (None, "whole", "head"):
            raise ValueError(f"qk_norm {qk_norm!r}: None, 'whole' or 'head'")
        self.qk_norm, self.norm_eps = qk_norm, float(norm_eps)
        self.q_temp = (float(q_temp[0]), int(q_temp[1])) if q_temp else None
        if self.q_temp and self.q_temp[1] <= 0:
            raise ValueError("the query temperature's period must be positive")
        self.sinks = bool(sinks)
        self.keep_first = int(keep_first) if self.window else 0
        if self.keep_first < 0:
            raise ValueError("a window keeps no negative number of first keys")
        self.maps, self.diff_init, self.head_gate = int(maps), float(diff_init), bool(head_gate)
        if self.maps not in (1, 2) or self.head_dim % self.maps:
            raise ValueError(f"{maps} maps in a key row of {head_dim}: one, or two equal halves")
        if self.head_gate and self.maps == 1:
            raise ValueError("a gate per head comes with two maps a head")
        if self.maps > 1 and (self.qkv_bias or self.score_cap or self.sinks or self.qk_norm
                              or self.q_temp or self.values_are_keys):
            raise ValueError("two maps a head go with plain projections and a plain softmax")
        # what the cache slot keeps: this layer's own mask unless told otherwise
        self.cache_window = self.window if cache_window == -1 else (int(cache_window) if cache_window else None)
        self.cache_keep_first = self.keep_first if cache_keep_first is None else int(cache_keep_first)
        self.diff_lambda = 0.0
        self.w_q_gate = None
        self.own_kv = bool(own_kv)
        self.out_gate = bool(out_gate)
        if self.out_gate and (self.head_gate or self.maps > 1 or not self.own_kv):
            raise ValueError("a gate per column goes with one map a head, no gate per head, and "
                             "a layer's own keys and values")
        if v_mix not in V_MIX_CODES:
            raise ValueError(f"v_mix {v_mix!r}: None, 'leave' or 'blend'")
        self.v_mix = v_mix
        if self.v_mix and (self.values_are_keys or not self.own_kv or self.maps > 1):
            raise ValueError("values mixed across layers are a layer's own projected values")
        self.v_lambda = 0.0
        # whether the number is stored: "yes", "maybe" (loaded when there, never used), "no"
        self.v_mix_stored = v_mix_stored or ("yes" if self.v_mix else "no")
        if self.v_mix_stored not in ("yes", "maybe", "no") or (self.v_mix and self.v_mix_stored != "yes"):
            raise ValueError("v_mix_stored: 'yes', 'maybe' or 'no'; a layer that mixes stores its number")
        if not self.own_kv and self.values_are_keys:
            raise ValueError("values that are keys are a layer's own")
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None
        self.w_q_norm = self.w_k_norm = self.sink = None
        self._alone: dict = {}

    @property
    def prepared(self) -> bool:
        """Whether q and k get more than a rotation between projection and cache (the kernels
        then take the projection in float32 and do all of it in one pass)."""
        return bool(self.values_are_keys or self.qk_norm or self.q_temp
                    or self.value_dim != self.head_dim or self.maps > 1 or self.out_gate
                    or self.v_mix)

    # ---- declarations

    def cache_spec(self) -> CacheSpec:
        value_dim = None if self.value_dim == self.head_dim else self.value_dim
        return CacheSpec(self.n_kv, self.head_dim, self.cache_window, value_dim,
                         keep_first=self.cache_keep_first if self.cache_window else 0)

    def _projections(self) -> list:
        """The stacked projections in order: (name key, rows)."""
        out = [("q", self.n_q * self.head_dim)]
        if not self.own_kv:
            return out
        out.append(("k", self.n_kv * self.head_dim))
        if not self.values_are_keys:
            out.append(("v", self.n_kv * self.value_dim))
        return out

    def param_specs(self) -> dict:
        h, n = self.hidden, self.names
        specs = {}
        for key, rows in self._projections():
            specs[f"{n[key]}.weight"] = TensorSpec((rows, h))
            if self.qkv_bias:
                specs[f"{n[key]}.bias"] = TensorSpec((rows,), role="vector")
        specs[f"{n['o']}.weight"] = TensorSpec((h, self.n_q * self.value_dim))
        if self.o_bias:
            specs[f"{n['o']}.bias"] = TensorSpec((h,), role="vector")
        if self.qk_norm:
            per = 1 if self.qk_norm == "head" else None
            specs[f"{n['q_norm']}.weight"] = TensorSpec(((per or self.n_q) * self.head_dim,),
                                                        role="vector", init="one_plus_normal")
            specs[f"{n['k_norm']}.weight"] = TensorSpec(((per or self.n_kv) * self.head_dim,),
                                                        role="vector", init="one_plus_normal")
        if self.out_gate:
            specs[f"{n['gate']}.weight"] = TensorSpec((self.n_q * self.value_dim, h))
        if self.v_mix_stored != "no":
            specs[n["v_mix"]] = TensorSpec((), role="vector", optional=self.v_mix_stored == "maybe")
        if self.sinks:
            specs[f"{n['sink']}.weight"] = TensorSpec((self.n_q,), role="vector")
        if self.maps > 1:
            for key in ("lq1", "lk1", "lq2", "lk2"):
                specs[n[key]] = TensorSpec((self.head_dim // self.maps,), role="vector")
        if self.head_gate:
            specs[f"{n['gate']}.weight"] = TensorSpec((self.n_q, h))
        return specs

    def bind(self, params, dtype, device) -> None:
        n = self.names
        # One projection for q, k and v: rows [q heads | k heads | v heads].
        keys = [key for key, _rows in self._projections()]
        stacked = [params[f"{n[key]}.weight"] for key in keys]
        if self.head_gate:
            # the gate's rows ride behind q, k, v in the same product; a layer that reads
            # another's keys and values projects [q | gate] only
            gate = params[f"{n['gate']}.weight"]
            stacked.append(gate)
            self.w_q_gate = torch.cat([stacked[0], gate], dim=0).contiguous()
        if self.out_gate:
            stacked.append(params[f"{n['gate']}.weight"])
        self.w_qkv = torch.cat(stacked, dim=0).contiguous()
        if self.v_mix:
            self.v_lambda = float(params[n["v_mix"]].float())
        if self.maps > 1:
            dot = lambda a, b: (params[n[a]].float() * params[n[b]].float()).sum()
            self.diff_lambda = float(torch.exp(dot("lq1", "lk1")) - torch.exp(dot("lq2", "lk2"))
                                     + self.diff_init)
        if self.qkv_bias:
            biases = [params[f"{n[key]}.bias"] for key in keys]
            common = torch.float32 if any(b.dtype == torch.float32 for b in biases) else dtype
            if self.out_gate:     # the gate's rows have no bias
                biases.append(torch.zeros(self.n_q * self.value_dim, dtype=common,
                                          device=biases[0].device))
            self.b_qkv = torch.cat([b.to(common) for b in biases]).contiguous()
        self.w_o = params[f"{n['o']}.weight"]
        self.b_o = params.get(f"{n['o']}.bias")
        if self.qk_norm:
            # both in float32: one dtype code for the two
            self.w_q_norm = params[f"{n['q_norm']}.weight"].float().contiguous()
            self.w_k_norm = params[f"{n['k_norm']}.weight"].float().contiguous()
        if self.sinks:
            self.sink = params[f"{n['sink']}.weight"].float().contiguous()
        self._alone.clear()

    def prepare(self, max_positions: int, device) -> None:
        self.position.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        total = 0
        for t in (self.w_qkv, self.b_qkv, self.w_o, self.b_o, self.w_q_norm, self.w_k_norm,
                  self.sink):   # (w_q_gate repeats rows of w_qkv)
            if t is not None:
                total += t.numel() * t.element_size()
        return total

    # ---- one step

    @property
    def lowerable(self) -> bool:
        """The host core runs this attention itself when the kernels can apply its position
        encoding."""
        return self.position.describe() is not None

    def lower(self, program, cache, state=None) -> None:
        pos = self.position.describe()
        if pos is None:
            raise ValueError("an attention whose position encoding applies itself is not lowered")
        if cache.k.dtype != self.w_qkv.dtype:
            raise ValueError("the kernels keep keys and values in the compute dtype")
        bias_code = lambda t: ops.dtype_code(t.dtype) if t is not None else ops.F32
        ptr = lambda t: 0 if t is None else t.data_ptr()
        w, b = self.w_qkv, self.b_qkv
        if cache.writes and not self.own_kv:
            raise ValueError("an attention without key and value projections reads a cache "
                             "another layer writes")
        if not cache.writes and self.own_kv:
            # Reads a cache another entry fills: only the queries are projected.
            rows = self.n_q * self.head_dim
            w, b = w[:rows], None if b is None else b[:rows]
            if self.head_gate:
                w = self.w_q_gate
            if self.out_gate or self.v_mix:
                raise ValueError("a gate per column and mixed values go with a cache the layer writes")
        if self.v_mix:
            # room in the step for what a "leave" layer hands to the "blend" layers after it
            program.need_carried(self.n_kv * self.value_dim)
        # (a kind of its own where the fixed-point stream's kernels would not do the same)
        program.append("attention_prepared" if self.prepared or self.sinks else "attention",
                       core.attention_params(
            w_qkv=w.data_ptr(), b_qkv=ptr(b), b_qkv_dtype=bias_code(b),
            w_o=self.w_o.data_ptr(), b_o=ptr(self.b_o), b_o_dtype=bias_code(self.b_o),
            n_q=self.n_q, n_kv=self.n_kv, head_dim=self.head_dim, rotary_dim=pos.rotary_dim,
            cos=ptr(pos.cos), sin=ptr(pos.sin),
            table_positions=0 if pos.cos is None else pos.cos.shape[0],
            interleaved=pos.interleaved, k_cache=cache.k.data_ptr(), v_cache=cache.v.data_ptr(),
            group=cache.group, page_size=cache.page_size, scale=self.scale,
            window=self.window or 0, writes=cache.writes, score_cap=self.score_cap,
            distance_slopes=ptr(pos.distance_slopes), sinks=ptr(self.sink),
            q_norm=ptr(self.w_q_norm), k_norm=ptr(self.w_k_norm), norm_dtype=ops.F32,
            norm_eps=self.norm_eps, temp_coef=self.q_temp[0] if self.q_temp else 0.0,
            temp_every=self.q_temp[1] if self.q_temp else 0,
            values_are_keys=self.values_are_keys,
            value_dim=self.value_dim if self.prepared else 0,
            keep_first=self.keep_first, maps=self.maps, head_gate=self.head_gate,
            diff_lambda=self.diff_lambda, diff_eps=self.norm_eps,
            diff_scale=1.0 - self.diff_init if self.maps > 1 else 1.0,
            head_norm=self.qk_norm == "head", out_gate=self.out_gate,
            v_mode=V_MIX_CODES[self.v_mix], v_lambda=self.v_lambda))

    def forward(self, x, step, cache, state, accum):
        if self.position.describe() is not None:
            # the operations `lower` appends, as a program of their own
            key = (cache.k.data_ptr(), cache.group, cache.writes)
            alone = self._alone.get(key)
            if alone is None:
                alone = self._alone[key] = OneOp(x.dtype, self.hidden, 0,
                                                 lambda program: self.lower(program, cache))
            _logits, _x, pending = alone.run(step, accum, x=x)
            return pending
        if self.prepared or self.sinks:
            raise ValueError("an attention with norms over q and k, a query temperature, sinks "
                             "or values that are keys needs a position encoding the kernels apply")
        # The encoding applies itself: project, let it transform q and k where they lie, then
        # write keys and values to the cache as they are.
        n_q, n_kv, d = self.n_q, self.n_kv, self.head_dim
        table = step.block_tables[cache.group]
        w, b = self.w_qkv, self.b_qkv
        if not cache.writes:
            w, b = w[:n_q * d], None if b is None else b[:n_q * d]
        k_cache, v_cache = (cache.k, cache.v) if cache.writes else (None, None)
        q = ops.linear(x, w, b)
        heads_kv = n_kv if cache.writes else 0
        q_part = q[:, :n_q * d].view(-1, n_q, d)
        k_part = q[:, n_q * d:(n_q + heads_kv) * d].view(-1, heads_kv, d) if heads_kv else None
        self.position.apply(q_part, k_part, step.positions)
        ops.rope_kv_write(q, None, None, step.positions, step.token_seq, table, k_cache,
                          v_cache, n_q, heads_kv, d, 0, cache.writes)
        attended = ops.attention(q, q.shape[1], cache.k, cache.v, step, table, n_q, n_kv, d,
                                 self.scale, self.window, score_cap=self.score_cap)
        return ops.project_into_stream(attended, self.w_o, self.b_o, accum)
