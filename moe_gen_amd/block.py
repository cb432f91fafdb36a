"""Shared machinery of the three MoE blocks: the SwiGLU MLP module, weight collection
(resident parameters, fp8 + block scales, or an engine that hands weights out slot by
slot) and the fused forward  router -> dispatch -> grouped SwiGLU -> combine."""
from __future__ import annotations

import torch
from torch import nn

from . import ops

FP8 = torch.float8_e4m3fn


class StageTimer:
    """Optional per-stage timing of a block's forward with events recorded on the stream the
    kernels are launched on (torch's current stream).  Attach as `block.stage_timer`."""

    def __init__(self):
        self.spans = []      # (name, start_event, end_event)

    class _Span:
        def __init__(self, timer, name):
            self.t, self.name = timer, name

        def __enter__(self):
            self.a = torch.cuda.Event(enable_timing=True)
            self.a.record()

        def __exit__(self, *exc):
            b = torch.cuda.Event(enable_timing=True)
            b.record()
            self.t.spans.append((self.name, self.a, b))

    def span(self, name):
        return StageTimer._Span(self, name)

    def totals_ms(self) -> dict:
        """name -> list of durations (ms); call after torch.cuda.synchronize()."""
        out = {}
        for name, a, b in self.spans:
            out.setdefault(name, []).append(a.elapsed_time(b))
        return out


class _NoSpan:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


def _span(timer, name):
    return timer.span(name) if timer is not None else _NoSpan()


def _grouped(timer, tag, x, row_map, ptrs, offsets, n_rows):
    """Both launches of the expert MLP; split (and timed per launch) when a timer is attached."""
    if timer is None:
        return ops.grouped_swiglu(x, row_map, ptrs, offsets, n_rows)
    act = torch.empty((n_rows, ptrs.inter), dtype=torch.bfloat16, device=x.device)
    y = torch.empty((n_rows, ptrs.hidden), dtype=torch.bfloat16, device=x.device)
    with timer.span(tag + "_gate_up"):
        ops.grouped_swiglu(x, row_map, ptrs, offsets, n_rows, act, y, ops.PHASE_GATE_UP)
    with timer.span(tag + "_down"):
        ops.grouped_swiglu(x, row_map, ptrs, offsets, n_rows, act, y, ops.PHASE_DOWN)
    return y


def _require_silu(config):
    act = getattr(config, "hidden_act", "silu")
    if act != "silu":
        raise NotImplementedError(f"expert activation {act!r}: only 'silu' (SwiGLU) is implemented")


def attach_fp8_weight(linear: nn.Linear, q: torch.Tensor, scale_inv: torch.Tensor) -> None:
    """Give an nn.Linear an fp8-e4m3fn weight with its 128x128 block scales, under the
    checkpoint's names `weight` / `weight_scale_inv` (the scale is multiplied, Wrapper.py:128)."""
    linear.weight = nn.Parameter(q, requires_grad=False)
    linear.weight_scale_inv = nn.Parameter(scale_inv, requires_grad=False)


class SwiGLUMLP(nn.Module):
    """down(silu(gate(x)) * up(x)) with three bias-free Linear layers.

    Same parameter tree as DeepseekV3MLP (modeling_deepseek_v3.py:439-467) /
    DeepseekV2MLP (:425-453); `names` lets Mixtral call them w1 / w3 / w2.
    Stand-alone calls run the grouped kernel with a single group."""

    names = ("gate_proj", "up_proj", "down_proj")

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        g, u, d = self.names
        setattr(self, g, nn.Linear(hidden_size, intermediate_size, bias=False))
        setattr(self, u, nn.Linear(hidden_size, intermediate_size, bias=False))
        setattr(self, d, nn.Linear(intermediate_size, hidden_size, bias=False))

    def projections(self):
        return tuple(getattr(self, n) for n in self.names)

    @torch.no_grad()
    def forward(self, x):
        shape = x.shape
        x2d = x.reshape(-1, shape[-1])
        if not x2d.is_contiguous():
            x2d = x2d.contiguous()
        n = x2d.shape[0]
        ptrs = collect_pointers([self], None)[0]
        offsets = torch.tensor([0, n], dtype=torch.int32, device=x.device)
        return ops.grouped_swiglu(x2d, None, ptrs, offsets, n).view(*shape)


def _unwrap(expert):
    """MoE-Gen replaces experts by Expert_Wrapper objects that keep the MLP in `.module`
    (Wrapper.py:449); accept both."""
    return getattr(expert, "module", expert)


def _tensors_of(expert, fetched=None):
    """(gate, up, down, s_gate, s_up, s_down) of one expert.

    fetched: optional dict `"<proj>.weight" -> tensor` obtained from an engine's get_weights();
    block scales come from the Linear's `weight_scale_inv` or, for a wrapped expert, from the
    wrapper's `weight_dequant_scale["<proj>.weight_scale_inv"]` (Wrapper.py:482-489)."""
    mlp = _unwrap(expert)
    wrap_scales = getattr(expert, "weight_dequant_scale", None) or {}
    ws, ss = [], []
    for name in mlp.names:
        lin = getattr(mlp, name)
        w = fetched[name + ".weight"] if fetched is not None else lin.weight.data
        s = wrap_scales.get(name + ".weight_scale_inv")
        if s is None:
            s = getattr(lin, "weight_scale_inv", None)
            s = None if s is None else s.data
        ws.append(w)
        ss.append(s)
    return (*ws, *ss)


def collect_pointers(experts, cache, counts=None):
    """Pointer tables for a list of expert modules, plus the list of engine keys to release
    once the kernels that read the weights are enqueued.

    counts: optional per-expert token counts (device int32 [E]).  When given and the engine can
    stage on demand (it has `fetch`), only the experts with a non-zero count are copied, busiest
    first, and the others get a placeholder pointer that no tile ever reads -- the reference
    copies every expert of the layer blindly (HtoD_Engine.cpp:201-268).  Costs one host read of
    E integers per call.

    Experts backed by an engine (an Expert_Wrapper-like object with `core_engine`,
    `get_weights=True` and `expert_weights_idx`) are fetched through
    `core_engine.get_weights(key)` exactly as Wrapper.py:479-491 does; the caller frees them
    with `free_weights_buffer(key)` (Wrapper.py:517).  Resident experts are cached in `cache`
    (a dict) keyed on the storage addresses of the first and last expert."""
    first = experts[0]
    engine_backed = bool(getattr(first, "get_weights", False)) and hasattr(first, "core_engine")
    if engine_backed:
        cols = [[] for _ in range(6)]
        keys = []
        # every expert of the layer is fetched below, so none of this layer's slots can be left
        # behind by a skipped expert; one call reclaims what the previous layer left
        if getattr(first, "expert_idx", -1) != -1:
            first.core_engine.clear_expert_buffer(first.layer_idx, 0)
        hot = None
        if counts is not None and hasattr(first.core_engine, "fetch"):
            c_host = counts.tolist()
            hot = sorted((e for e in range(len(experts)) if c_host[e] > 0), key=lambda e: -c_host[e])
            first.core_engine.fetch([experts[e].expert_weights_idx for e in hot])
        if hot is None:
            chosen = range(len(experts))
        else:
            chosen = hot or [0]                  # no routed token at all: one expert stands in
        got = {}
        for e in chosen:
            ex = experts[e]
            fetched = ex.core_engine.get_weights(ex.expert_weights_idx)
            keys.append((ex.core_engine, ex.expert_weights_idx))
            got[e] = _tensors_of(ex, fetched)
        stand_in = got[next(iter(chosen))]
        for e in range(len(experts)):
            for c, t in zip(cols, got.get(e, stand_in)):
                c.append(t)
        fp8 = cols[0][0].dtype == FP8
        p = ops.expert_pointers(cols[0], cols[1], cols[2], *(cols[3:] if fp8 else (None, None, None)))
        return p, keys
    f = _tensors_of(first)
    last = _tensors_of(experts[-1])
    stamp = (len(experts), f[0].data_ptr(), f[0].dtype, tuple(f[0].shape), last[2].data_ptr())
    if cache is not None and cache.get("stamp") == stamp:
        return cache["ptrs"], []
    cols = [[] for _ in range(6)]
    for ex in experts:
        for c, t in zip(cols, _tensors_of(ex)):
            c.append(t)
    fp8 = cols[0][0].dtype == FP8
    p = ops.expert_pointers(cols[0], cols[1], cols[2], *(cols[3:] if fp8 else (None, None, None)))
    if cache is not None:
        cache["stamp"], cache["ptrs"] = stamp, p
    return p, []


def _gate_weight_bf16(weight: torch.Tensor, cache: dict) -> torch.Tensor:
    """The router kernel reads the gate matrix as bf16.  MoE-Gen delivers it in bf16; an fp32
    parameter is accepted only if every entry is exactly representable in bf16."""
    w = weight.data
    if w.dtype == torch.bfloat16:
        return w if w.is_contiguous() else w.contiguous()
    key = (w.data_ptr(), w._version)
    if cache.get("gate_key") != key:
        wb = w.to(torch.bfloat16)
        if not torch.equal(wb.to(w.dtype), w):
            raise NotImplementedError("gate weight is not representable in bf16; the fused router reads bf16")
        cache["gate_key"], cache["gate_bf16"] = key, wb.contiguous()
    return cache["gate_bf16"]


@torch.no_grad()
def moe_forward(block, hidden_states: torch.Tensor, spec: ops.RouterSpec, gate_weight: torch.Tensor,
                bias, experts, shared, combine_mode: int, want_logits: bool = False):
    """The whole layer for one call.  Returns (out [same shape as hidden_states], logits | None)."""
    if not hidden_states.is_cuda:
        raise RuntimeError("MoE block called on a CPU tensor: this implementation runs on the GPU only")
    if hidden_states.dtype != torch.bfloat16:
        raise TypeError(f"hidden_states must be bfloat16, got {hidden_states.dtype}")
    shape = hidden_states.shape
    x = hidden_states.reshape(-1, shape[-1])
    if not x.is_contiguous():
        x = x.contiguous()
    n, h = x.shape
    k, E = spec.top_k, spec.n_experts
    residual = None
    fuse = getattr(block, "_norm_residual", None)
    timer = getattr(block, "stage_timer", None)
    if fuse is not None:                      # see norm_moe_residual
        residual = x
        with _span(timer, "rmsnorm"):
            x = ops.rmsnorm(x, fuse[0], fuse[1])
    cache = block.__dict__.setdefault("_moe_cache", {})
    gw = _gate_weight_bf16(gate_weight, cache)
    b = None if bias is None else bias.data.to(torch.float32)
    with _span(timer, "router"):
        idx, w, logits = ops.router(x, gw, b, spec, want_logits)
    block.last_topk_idx, block.last_topk_weight = idx, w
    fused_gather = getattr(block, "fused_gather", True)
    with _span(timer, "dispatch"):
        counts, offsets, perm, pos, xs = ops.dispatch(idx, E, None if fused_gather else x)
        row_map = torch.div(perm, k, rounding_mode="floor").to(torch.int32) if fused_gather else None
    block.last_counts = counts
    aware = counts if getattr(block, "routing_aware_staging", False) else None
    ptrs, keys = collect_pointers(list(experts), cache.setdefault("routed", {}), aware)
    y = _grouped(timer, "routed", x if fused_gather else xs, row_map, ptrs, offsets, n * k)
    for eng, key in keys:
        eng.free_weights_buffer(key)
    sh = None
    if shared is not None:
        sp, skeys = collect_pointers([shared], cache.setdefault("shared", {}))
        so = cache.get("shared_off")
        if so is None or so[0] != n or so[1].device != x.device:
            so = (n, torch.tensor([0, n], dtype=torch.int32, device=x.device))
            cache["shared_off"] = so
        sh = _grouped(timer, "shared", x, None, sp, so[1], n)
        for eng, key in skeys:
            eng.free_weights_buffer(key)
    with _span(timer, "combine"):
        out = ops.combine(y, pos, idx, w, sh, combine_mode, residual=residual)
    return out.view(*shape), logits


@torch.no_grad()
def norm_moe_residual(block, hidden_states: torch.Tensor, norm_weight: torch.Tensor, eps: float = 1e-6):
    """The MLP half of the reference decoder layer around an MoE block
    (modeling_deepseek_v3.py:1361-1365, modeling_deepseek_v2.py:1522-1526):

        residual = hidden_states
        hidden_states = post_attention_layernorm(hidden_states)
        hidden_states = mlp(hidden_states)
        hidden_states = residual + hidden_states

    with the norm as one kernel and the residual add folded into the combine's output pass.
    Returns what `block(...)` returns with the new residual stream in place of the block output
    (Mixtral: a tuple with the router logits second)."""
    w = norm_weight.data if isinstance(norm_weight, torch.nn.Parameter) else norm_weight
    block._norm_residual = (w, float(eps))
    try:
        return block(hidden_states)
    finally:
        block._norm_residual = None
