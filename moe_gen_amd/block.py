"""Shared machinery of the three MoE blocks: the SwiGLU MLP module, weight collection
(resident parameters, fp8 + block scales, or an engine that hands weights out slot by
slot, in waves when its pool is smaller than the layer) and the fused forward
router -> dispatch -> grouped SwiGLU -> combine."""
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
        if engine_backed(self):
            raise RuntimeError("SwiGLUMLP.forward: engine-backed weights are handled by the MoE block")
        ptrs = collect_pointers([self], None)
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
    if fetched is not None:                     # hot path of the staged walk: no attribute look-ups on the modules
        keys = expert.__dict__.get("_moe_keys")
        if keys is None:                        # the tensor names of this expert, built once
            names = _unwrap(expert).names
            keys = (tuple(n + ".weight" for n in names), tuple(n + ".weight_scale_inv" for n in names))
            expert.__dict__["_moe_keys"] = keys
        wk, sk = keys
        w0 = fetched[wk[0]]
        if w0.dtype != FP8:
            return (w0, fetched[wk[1]], fetched[wk[2]], None, None, None)
        wrap_scales = expert.__dict__.get("weight_dequant_scale")
        if wrap_scales:
            return (w0, fetched[wk[1]], fetched[wk[2]], wrap_scales.get(sk[0]), wrap_scales.get(sk[1]), wrap_scales.get(sk[2]))
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


def _pointer_table(rows):
    """ExpertPointers from a list of (gate, up, down, s_gate, s_up, s_down) tuples."""
    cols = list(zip(*rows))
    fp8 = cols[0][0].dtype == FP8
    return ops.expert_pointers(list(cols[0]), list(cols[1]), list(cols[2]),
                               *((list(c) for c in cols[3:]) if fp8 else (None, None, None)))


def engine_backed(expert) -> bool:
    """Whether an expert's weights come from an engine call by call: an Expert_Wrapper-like object
    with `core_engine`, `get_weights=True` and `expert_weights_idx` (Wrapper.py:437-468)."""
    return bool(getattr(expert, "get_weights", False)) and hasattr(expert, "core_engine")


def collect_pointers(experts, cache):
    """Pointer tables for a list of RESIDENT expert modules, cached in `cache` (a dict) keyed on
    the storage addresses of the first and last expert."""
    f = _tensors_of(experts[0])
    last = _tensors_of(experts[-1])
    stamp = (len(experts), f[0].data_ptr(), f[0].dtype, tuple(f[0].shape), last[2].data_ptr())
    if cache is not None and cache.get("stamp") == stamp:
        return cache["ptrs"]
    p = _pointer_table([_tensors_of(ex) for ex in experts])
    if cache is not None:
        cache["stamp"], cache["ptrs"] = stamp, p
    return p


def pool_size(expert, module_type: str = "routed_expert") -> int:
    """How many modules of `module_type` the engine behind `expert` can hold at once.

    The library's Stager reports it (`pool_size`).  MoE-Gen's engine keeps it in the config the
    wrapper carries: `engine_config.GPU_Buffer_Config.num_prefill_module_buffer[type]`, or
    `num_decoding_module_buffer[type]` once `Expert_Wrapper.phase` is "decoding"
    (deepseekv3_initializer.py:912-927, Wrapper.py:435).  Unknown: 1, the reference's own pattern
    of one expert at a time (Wrapper.py:475-521)."""
    eng = expert.core_engine
    if callable(getattr(eng, "pool_size", None)):
        return max(1, int(eng.pool_size(module_type)))
    gb = getattr(getattr(expert, "engine_config", None), "GPU_Buffer_Config", None)
    if gb is not None:
        decoding = getattr(type(expert), "phase", "prefill") == "decoding"
        table = gb.num_decoding_module_buffer if decoding else gb.num_prefill_module_buffer
        if table and module_type in table:
            return max(1, int(table[module_type]))
    return 1


def expert_waves(n_experts: int, pool: int, hot=None, backed=None):
    """Cut a layer's experts into waves for a pool of `pool` slots.

    Returns a list of (first, last_plus_one, fetch_list): the grouped kernels of a wave run on the
    experts [first, last_plus_one) and `fetch_list` names the ones whose weights the wave holds.
    Experts that fit the pool at once are one wave.  Otherwise a wave takes HALF the pool, so that the
    engine copies the next wave into the other half while this one is multiplied -- the overlap the
    reference gets from fetching, using and freeing one expert at a time against a pool that its copy
    worker keeps filling (Wrapper.py:475-521, HtoD_Engine.cpp:201-268); with waves as large as the pool
    every copy would wait for a release and every launch for a copy.
    Without `hot` every expert is fetched, in id order -- the order in which the copy worker delivers
    them, so a wave's weights are exactly what the pool holds or receives next.  With `hot` (ids of the
    experts that received tokens, on-demand staging) only those are fetched; a wave then spans from its
    first to its last hot expert and the cold ones in between own no rows.
    `backed` (ids of the experts whose weights come from the engine; the others are resident, the
    reference decides expert by expert, deepseekv3_initializer.py:1259-1266) restricts the fetch lists
    to those ids, and the waves then cover every expert: the first starts at expert 0, each ends where
    the next one starts and the last at n_experts, so that resident experts run in the wave they fall into."""
    pool = max(1, int(pool))
    ids = list(range(n_experts)) if hot is None else sorted(hot)
    if backed is not None:
        keep = set(backed)
        ids = [e for e in ids if e in keep]
    step = pool if len(ids) <= pool else max(1, pool // 2)
    waves = [(ids[i], ids[min(i + step, len(ids)) - 1] + 1, ids[i:i + step]) for i in range(0, len(ids), step)]
    if backed is None:
        return waves
    if not waves:
        return [(0, n_experts, [])]
    starts = [0] + [w[0] for w in waves[1:]] + [n_experts]
    return [(starts[i], starts[i + 1], w[2]) for i, w in enumerate(waves)]


def staged_experts_forward(experts, launch, counts_host=None, on_demand=False, stream_wait=None, module_type="routed_expert"):
    """Run a layer's engine-backed experts through a pool that may be smaller than the layer.

    Per wave (expert_waves): get_weights for the wave's experts, `launch(rows, first, last, n_rows)`
    enqueues the grouped kernels for experts [first, last) with `rows[i]` the weight tensors of
    expert first+i, then the wave's slots are released -- at once when the engine orders the
    release on the stream itself (`stream_ordered_release`, the library's Stager), otherwise after
    `stream_wait()` has drained the compute stream: the reference's pool marks a slot free on the
    host and its copy thread overwrites it immediately (GPU_Weight_Buffer.cpp:163-169), which is
    why Expert_Wrapper synchronises before free_weights_buffer (Wrapper.py:512-517).

    Experts are taken one by one (the reference wraps every expert and sets `get_weights` per expert,
    Mixtral_Initializer.py:761-787, deepseekv3_initializer.py:1259-1266): one with `get_weights`
    false keeps its weights resident and runs in the wave its id falls into.

    counts_host: per-expert token counts on the host; needed when there is more than one wave (the
    launch of a wave is sized by its own rows) and for on-demand staging.
    on_demand: fetch only experts with tokens through the engine's `fetch` (busiest first when
    they fit the pool at once)."""
    E = len(experts)
    backed = [e for e in range(E) if engine_backed(experts[e])]
    if not backed:
        raise RuntimeError("staged_experts_forward: no expert of the layer takes its weights from an engine")
    mixed = len(backed) < E
    first = experts[backed[0]]
    eng = first.core_engine
    pool = pool_size(first, module_type)
    routed = getattr(first, "expert_idx", -1) != -1
    if routed:
        # every expert of the layer is fetched (or never copied, on demand), so none of this layer's
        # slots is left behind by a skipped expert; one call reclaims what the previous layer left
        eng.clear_expert_buffer(first.layer_idx, 0)
    hot = None
    if on_demand and counts_host is not None and hasattr(eng, "fetch"):
        hot = [e for e in backed if counts_host[e] > 0]
        if not hot and not mixed:
            return
        if hot and len(hot) <= pool:
            hot_by_load = sorted(hot, key=lambda e: -counts_host[e])
            eng.fetch([experts[e].expert_weights_idx for e in hot_by_load])
    waves = expert_waves(E, pool, hot, backed if mixed else None)
    if len(waves) > 1 and counts_host is None:
        raise RuntimeError("staged_experts_forward: more than one wave needs the per-expert counts on the host")
    ordered = bool(getattr(eng, "stream_ordered_release", False))
    on_demand_waves = hot is not None and len(hot) > pool
    # a wave is half the pool, so the next wave's copies go into the half this wave does not hold; a pool of a
    # single slot has no other half, and its next copy can only be asked for once the slot has been let go
    ahead = on_demand_waves and all(len(a[2]) + len(b[2]) <= pool for a, b in zip(waves, waves[1:]))
    if on_demand_waves and ahead:                            # the first wave's copies; each wave then asks for the next one's
        eng.fetch([experts[e].expert_weights_idx for e in waves[0][2]])
    resident_rows = {e: _tensors_of(experts[e]) for e in range(E) if e not in set(backed)} if mixed else {}
    for w, (a, b, fetch) in enumerate(waves):
        if on_demand_waves:
            if not ahead:
                eng.fetch([experts[e].expert_weights_idx for e in fetch])
            elif w + 1 < len(waves):
                eng.fetch([experts[e].expert_weights_idx for e in waves[w + 1][2]])
        got = {e: _tensors_of(experts[e], eng.get_weights(experts[e].expert_weights_idx)) for e in fetch}
        got.update({e: resident_rows[e] for e in range(a, b) if e in resident_rows})
        if not got:                                          # nothing but engine-backed experts without rows
            continue
        stand_in = next(iter(got.values()))                  # an expert without rows is never read
        rows = [got.get(e, stand_in) for e in range(a, b)]
        n_rows = None if counts_host is None else int(sum(counts_host[a:b]))
        launch(rows, a, b, n_rows)
        if not ordered and stream_wait is not None and fetch:
            stream_wait()
        for e in fetch:
            eng.free_weights_buffer(experts[e].expert_weights_idx)


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


def _engine_experts(block, timer, tag, experts, a_rows, row_map, offsets, n_rows, counts):
    """The expert MLPs of one layer with weights handed out by an engine, wave by wave."""
    first = next(ex for ex in experts if engine_backed(ex))
    routed = tag == "routed"
    mtype = "routed_expert" if routed else "shared_expert"
    E = len(experts)
    aware = routed and bool(getattr(block, "routing_aware_staging", False)) and hasattr(first.core_engine, "fetch")
    counts_host = None
    n_backed = sum(1 for ex in experts if engine_backed(ex))
    if routed and (aware or pool_size(first, mtype) < n_backed):
        counts_host = counts.tolist()                        # one read of E integers (the reference reads them too, :673)
    hidden, inter = a_rows.shape[1], None
    act = y = None
    stream = torch.cuda.current_stream().cuda_stream       # looked up once per layer call, not per wave
    checked = False

    def launch(rows, a, b, rows_in_wave):
        nonlocal act, y, inter, checked
        ptrs = ops.expert_pointers_of_rows(rows, a_rows.device)
        if y is None:
            inter = ptrs.inter
            act = torch.empty((n_rows, inter), dtype=torch.bfloat16, device=a_rows.device)
            y = torch.empty((n_rows, hidden), dtype=torch.bfloat16, device=a_rows.device)
        bound = n_rows if rows_in_wave is None else rows_in_wave
        if not 0 <= bound <= n_rows:
            raise ValueError(f"rows of the wave {bound} outside [0, {n_rows}]")
        off = offsets[a:b + 1]
        if timer is None:       # (the first wave validates the layer's buffers; the later ones pass the same)
            ops.grouped_swiglu(a_rows, row_map, ptrs, off, n_rows, act, y, rows_bound=bound, checked=checked, stream=stream)
            checked = True
        else:
            with timer.span(tag + "_gate_up"):
                ops.grouped_swiglu(a_rows, row_map, ptrs, off, n_rows, act, y, ops.PHASE_GATE_UP, rows_bound=bound)
            with timer.span(tag + "_down"):
                ops.grouped_swiglu(a_rows, row_map, ptrs, off, n_rows, act, y, ops.PHASE_DOWN, rows_bound=bound)

    staged_experts_forward(experts, launch, counts_host, aware,
                           stream_wait=lambda: torch.cuda.current_stream().synchronize(), module_type=mtype)
    if y is None:                                            # no expert received a token
        y = torch.empty((n_rows, hidden), dtype=torch.bfloat16, device=a_rows.device)
    return y


def _shared_joins_routed(block, experts, shared, n, k, fused_gather, cache):
    """Whether this call runs the shared expert as one more group of the routed experts' grouped call, and if so the
    pointer tables of the 1 + E groups and the offset / row-map buffers of the joint call (cached per token count).

    It does when the shared expert alone would leave most CUs without a tile -- (n / 256 + 1) row tiles times I / 128
    column tiles fewer than 3/8 of the device's CUs: DeepSeek-V3 up to 1024 tokens, where the step gains 2-5 %; from
    2048 tokens on a launch pair of its own, with 256-row tiles, is the faster by 0.6 % -- and has the routed experts'
    shapes and dtype (one shared expert: DeepSeek-V3 / R1; DeepSeek-V2's two are one MLP of twice the width), with all
    weights resident.  `block.join_shared = False` keeps the two calls apart."""
    if shared is None or not fused_gather or not getattr(block, "join_shared", True):
        return None
    if engine_backed(shared) or any(engine_backed(ex) for ex in experts):
        return None
    E = len(experts)
    fit = cache.get("joint_fit")
    if fit is None or fit[0] != (id(shared), id(experts[0]), E):
        ts, tr = _tensors_of(shared), _tensors_of(experts[0])
        same = ts[0].shape == tr[0].shape and ts[0].dtype == tr[0].dtype and ts[2].shape == tr[2].shape
        dev = ts[0].device
        fit = ((id(shared), id(experts[0]), E), same, -(-ts[0].shape[0] // 128), dev,
               torch.cuda.get_device_properties(dev).multi_processor_count)
        cache["joint_fit"] = fit
    _, same, col_tiles, dev, cus = fit
    if not same or (n // 256 + 1) * col_tiles * 8 >= 3 * cus:
        return None
    ptrs = collect_pointers([shared] + experts, cache.setdefault("shared+routed", {}))
    bufs = cache.get("joint")
    if bufs is None or bufs[0] != (n, k, E, dev):
        off = torch.zeros(E + 2, dtype=torch.int32, device=dev)        # [0, n, n + routed offsets 1 .. E]
        rows = torch.empty(n + n * k, dtype=torch.int32, device=dev)   # [0 .. n-1, routed row map]
        rows[:n] = torch.arange(n, dtype=torch.int32, device=dev)
        bufs = ((n, k, E, dev), off, rows)
        cache["joint"] = bufs
    return ptrs, bufs[1], bufs[2]


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
    cache = block.__dict__.setdefault("_moe_cache", {})
    gw = _gate_weight_bf16(gate_weight, cache)
    b = None if bias is None else bias.data.to(torch.float32)
    if fuse is not None:                      # see norm_moe_residual: the router reads x through the norm
        residual = x
        with _span(timer, "router"):
            idx, w, logits, x = ops.router(x, gw, b, spec, want_logits, norm_weight=fuse[0], eps=fuse[1])
    else:
        with _span(timer, "router"):
            idx, w, logits = ops.router(x, gw, b, spec, want_logits)
    block.last_topk_idx, block.last_topk_weight = idx, w
    fused_gather = getattr(block, "fused_gather", True)
    experts = list(experts)
    joined = _shared_joins_routed(block, experts, shared, n, k, fused_gather, cache)
    if joined is not None:
        # The shared expert as one more group of the routed call: all n token rows IN FRONT of the n*k routed rows
        # (identity entries at the head of the row map, written once; the routed offsets shifted by n).  Its tiles
        # then fill the CUs next to the routed experts' instead of a launch pair of their own that has a tile for a
        # fraction of them -- in front, because they are the tallest of the call and would be its tail at the end.
        ptrs_all, off_all, map_all = joined
        with _span(timer, "dispatch"):
            d = ops.dispatch(idx, E, None, out_row_map=map_all[n:])
            torch.add(d.offsets, n, out=off_all[1:])
        block.last_counts = d.counts
        y_all = _grouped(timer, "routed", x, map_all, ptrs_all, off_all, n * k + n)
        with _span(timer, "combine"):
            out = ops.combine(y_all[n:], d.pos, idx, w, y_all[:n], combine_mode, residual=residual)
        return out.view(*shape), logits
    with _span(timer, "dispatch"):
        d = ops.dispatch(idx, E, None if fused_gather else x, want_row_map=fused_gather)
    counts, offsets, pos, row_map = d.counts, d.offsets, d.pos, d.row_map
    block.last_counts = counts
    a_rows = x if fused_gather else d.xs
    if any(engine_backed(ex) for ex in experts):   # decided expert by expert, as the reference's initializers do
        y = _engine_experts(block, timer, "routed", experts, a_rows, row_map, offsets, n * k, counts)
    else:
        y = _grouped(timer, "routed", a_rows, row_map, collect_pointers(experts, cache.setdefault("routed", {})),
                     offsets, n * k)
    sh = None
    if shared is not None:
        so = cache.get("shared_off")
        if so is None or so[0] != n or so[1].device != x.device:
            so = (n, torch.tensor([0, n], dtype=torch.int32, device=x.device))
            cache["shared_off"] = so
        if engine_backed(shared):
            sh = _engine_experts(block, timer, "shared", [shared], x, None, so[1], n, None)
        else:
            sh = _grouped(timer, "shared", x, None, collect_pointers([shared], cache.setdefault("shared", {})), so[1], n)
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

    with the norm folded into the router's read of the rows (its normalised copy is a side output
    that the expert GEMMs read) and the residual add folded into the combine's output pass.
    Returns what `block(...)` returns with the new residual stream in place of the block output
    (Mixtral: a tuple with the router logits second)."""
    w = norm_weight.data if isinstance(norm_weight, torch.nn.Parameter) else norm_weight
    block._norm_residual = (w, float(eps))
    try:
        return block(hidden_states)
    finally:
        block._norm_residual = None
