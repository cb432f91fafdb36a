"""Operators of the MoE hot path on torch tensors: thin wrappers that validate shapes on
the host, allocate outputs with torch, and call the C ABI on torch's current stream."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import NamedTuple

import torch

from . import _native as N

SCORE = {"softmax": 0, "sigmoid": 1}
METHOD = {"greedy": 0, "group_limited_greedy": 1, "noaux_tc": 2}
COMBINE_F32, COMBINE_BF16_PROD, COMBINE_BF16_SEQ = 0, 1, 2


@dataclass
class RouterSpec:
    """Routing rules of one gate (the hyper-parameters MoEGate reads from its config)."""
    n_experts: int
    top_k: int
    scoring: str = "softmax"
    method: str = "greedy"
    n_group: int = 1
    topk_group: int = 1
    norm_topk_prob: bool = False
    scale_mode: int = 1               # 0 never, 1 only when not normalising (V2), 2 always (V3)
    routed_scaling_factor: float = 1.0
    norm_eps: float = 1e-20
    logits_bf16: bool = False         # Mixtral: the gate Linear runs in bf16
    weights_bf16: bool = False        # Mixtral: routing weights cast to bf16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, dtype, name: str, shape=None):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); this package has no CPU path")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def router(x: torch.Tensor, gate_w: torch.Tensor, bias, spec: RouterSpec, want_logits: bool = False,
           norm_weight: torch.Tensor | None = None, eps: float = 1e-6):
    """x bf16 [n,h], gate_w bf16 [E,h], bias fp32 [E] | None ->
    (topk_idx int32 [n,k], topk_weight fp32 [n,k], logits fp32 [n,E] | None).

    With norm_weight (bf16 [h]) the rows of x are raw hidden states read through the decoder
    layer's RMSNorm inside the same kernel, and a fourth result holds the normalised rows
    (bf16 [n,h]) -- bit-identical to rmsnorm() followed by router()."""
    n, h = x.shape
    E, k = spec.n_experts, spec.top_k
    _need(x, torch.bfloat16, "x")
    _need(gate_w, torch.bfloat16, "gate weight", (E, h))
    if bias is not None:
        _need(bias, torch.float32, "e_score_correction_bias", (E,))
    if spec.scoring not in SCORE:
        raise NotImplementedError(f"insupportable scoring function for MoE gating: {spec.scoring}")
    if spec.method not in METHOD:
        raise NotImplementedError(f"insupportable TopK function for MoE gating: {spec.method}")
    if spec.method == "noaux_tc" and bias is None:
        raise ValueError("noaux_tc routing needs e_score_correction_bias")
    idx = torch.empty((n, k), dtype=torch.int32, device=x.device)
    w = torch.empty((n, k), dtype=torch.float32, device=x.device)
    lg = torch.empty((n, E), dtype=torch.float32, device=x.device) if want_logits else None
    p = N.RouterParams(n, h, E, k, spec.n_group or 1, spec.topk_group or 1, SCORE[spec.scoring],
                       METHOD[spec.method], int(spec.norm_topk_prob), spec.scale_mode,
                       int(spec.logits_bf16), int(spec.weights_bf16), spec.norm_eps,
                       spec.routed_scaling_factor)
    if norm_weight is not None:
        _need(norm_weight, torch.bfloat16, "norm weight", (h,))
        xn = torch.empty_like(x)
        N.check(N.lib().moe_router_rmsnorm(_ptr(x), _ptr(norm_weight), float(eps), _ptr(gate_w), _ptr(bias),
                                           ctypes.byref(p), _ptr(xn), _ptr(idx), _ptr(w), _ptr(lg), _stream()),
                "moe_router_rmsnorm")
        return idx, w, lg, xn
    N.check(N.lib().moe_router(_ptr(x), _ptr(gate_w), _ptr(bias), ctypes.byref(p), _ptr(idx), _ptr(w),
                               _ptr(lg), _stream()), "moe_router")
    return idx, w, lg


class Dispatch(NamedTuple):
    counts: torch.Tensor             # int32 [E]
    offsets: torch.Tensor            # int32 [E+1]
    perm: torch.Tensor               # int32 [n*k]
    pos: torch.Tensor                # int32 [n*k]
    xs: torch.Tensor | None          # bf16 [n*k,h] gathered rows (only when x was given)
    row_map: torch.Tensor | None     # int32 [n*k] = perm // k (only when asked for)


def dispatch(topk_idx: torch.Tensor, n_experts: int, x: torch.Tensor | None = None, want_row_map: bool = False,
             out_row_map: torch.Tensor | None = None):
    """topk_idx int32 [n,k] -> Dispatch(counts [E], offsets [E+1], perm [n*k], pos [n*k], xs, row_map):
    if x bf16 [n,h] is given, xs holds the gathered rows [n*k,h]; with want_row_map, row_map[r] is
    the token row behind sorted row r (the grouped GEMM gathers through it).
    out_row_map: an int32 device buffer of at least n*k entries to write the row map into (its first n*k entries; a
    caller that adds groups of its own to the grouped call passes a slice of a longer map); it is returned as given."""
    _need(topk_idx, torch.int32, "topk_idx")
    n, k = topk_idx.shape
    dev = topk_idx.device
    counts = torch.empty(n_experts, dtype=torch.int32, device=dev)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(n * k, dtype=torch.int32, device=dev)
    pos = torch.empty(n * k, dtype=torch.int32, device=dev)
    if out_row_map is not None:
        _need(out_row_map, torch.int32, "out_row_map")
        if out_row_map.numel() < n * k:
            raise ValueError(f"out_row_map holds {out_row_map.numel()} entries, {n * k} needed")
        want_row_map = True
    row_map = out_row_map if out_row_map is not None else (
        torch.empty(n * k, dtype=torch.int32, device=dev) if want_row_map else None)
    xs, h = None, 0
    if x is not None:
        _need(x, torch.bfloat16, "x")
        if x.shape[0] != n:
            raise ValueError(f"x has {x.shape[0]} rows, topk_idx {n}")
        h = x.shape[1]
        xs = torch.empty((n * k, h), dtype=torch.bfloat16, device=dev)
    wsb = N.lib().moe_dispatch_workspace_bytes(n, k, n_experts)
    ws = torch.empty(wsb, dtype=torch.uint8, device=dev)
    N.check(N.lib().moe_dispatch(_ptr(topk_idx), n, k, n_experts, _ptr(counts), _ptr(offsets), _ptr(perm),
                                 _ptr(pos), _ptr(row_map), _ptr(x), h, _ptr(xs), _ptr(ws), wsb, _stream()),
            "moe_dispatch")
    return Dispatch(counts, offsets, perm, pos, xs, row_map)


@dataclass
class ExpertPointers:
    """Device arrays of per-expert weight (and block-scale) pointers, in the layout the
    grouped kernels read.  `keep` pins the tensors the pointers refer to."""
    n_experts: int
    hidden: int
    inter: int
    fp8: bool
    w_gate: torch.Tensor
    w_up: torch.Tensor
    w_down: torch.Tensor
    s_gate: torch.Tensor | None = None
    s_up: torch.Tensor | None = None
    s_down: torch.Tensor | None = None
    keep: tuple = ()


def expert_pointers(gates, ups, downs, s_gates=None, s_ups=None, s_downs=None, device=None) -> ExpertPointers:
    """Build pointer tables from lists of per-expert tensors: gate/up [I,h], down [h,I]
    (bf16, or float8_e4m3fn with fp32 scales [ceil(r/128), ceil(c/128)])."""
    E = len(gates)
    I, h = gates[0].shape
    fp8 = gates[0].dtype == torch.float8_e4m3fn
    want = torch.float8_e4m3fn if fp8 else torch.bfloat16
    for i in range(E):
        _need(gates[i], want, f"experts[{i}].gate weight", (I, h))
        _need(ups[i], want, f"experts[{i}].up weight", (I, h))
        _need(downs[i], want, f"experts[{i}].down weight", (h, I))
    dev = device or gates[0].device

    def table(ts):
        return torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64).to(dev, non_blocking=False)

    sg = su = sd = None
    if fp8:
        if s_gates is None or s_ups is None or s_downs is None:
            raise ValueError("fp8 expert weights need their *_scale_inv block scales")
        bi, bh = -(-I // 128), -(-h // 128)
        for i in range(E):
            _need(s_gates[i], torch.float32, f"experts[{i}].gate scale", (bi, bh))
            _need(s_ups[i], torch.float32, f"experts[{i}].up scale", (bi, bh))
            _need(s_downs[i], torch.float32, f"experts[{i}].down scale", (bh, bi))
        sg, su, sd = table(s_gates), table(s_ups), table(s_downs)
    keep = (tuple(gates), tuple(ups), tuple(downs), tuple(s_gates or ()), tuple(s_ups or ()), tuple(s_downs or ()))
    return ExpertPointers(E, h, I, fp8, table(gates), table(ups), table(downs), sg, su, sd, keep)


def _upload_words(values, device) -> torch.Tensor:
    """A device int64 array holding `values`, written by moe_write_words: the words travel in kernel arguments on
    the current stream: no pinned staging buffer to recycle, and nothing queued on the copy engine behind the weight
    copies that a stager keeps in flight there."""
    n = len(values)
    dev = torch.empty(n, dtype=torch.int64, device=device)
    arr = (ctypes.c_uint64 * n)(*values)
    if dev.device.index == torch.cuda.current_device():
        N.check(N.lib().moe_write_words(dev.data_ptr(), arr, n, _stream()), "moe_write_words")
    else:
        with torch.cuda.device(dev.device):
            N.check(N.lib().moe_write_words(dev.data_ptr(), arr, n, _stream()), "moe_write_words")
    return dev


_table_cache: dict = {}       # (device, shape, dtype, pointers) -> ExpertPointers of a wave seen before
_TABLE_CACHE_MAX = 32768


def expert_pointers_of_rows(rows, device) -> ExpertPointers:
    """Pointer tables for one wave of engine-delivered experts: `rows[i]` = (gate, up, down[, s_gate, s_up, s_down])
    of expert i.  The hot form of expert_pointers: shapes and dtypes are checked against the first expert's, all
    tables are written by ONE small launch that carries them in its arguments (six synchronous copies otherwise: 26
    waves of a DeepSeek-V3 layer cost 2.4 ms of host time that way), and the tables are slices of that one device
    array."""
    E = len(rows)
    g0, u0, d0 = rows[0][0], rows[0][1], rows[0][2]
    I, h = g0.shape
    fp8 = g0.dtype == torch.float8_e4m3fn
    want = torch.float8_e4m3fn if fp8 else torch.bfloat16
    gs, ds = (I, h), (h, I)
    if not g0.is_cuda:
        raise RuntimeError(f"expert weights must live on the GPU (got {g0.device}); this package has no CPU path")
    ncol = 6 if fp8 else 3
    vals = []
    for c in range(ncol):
        for r in rows:
            vals.append(r[c].data_ptr())
    # Slot addresses recur from call to call (an engine's pool is a fixed set of buffers, block scales are
    # resident): a wave whose pointers were all seen before, for tensors of this shape, reuses its device table.
    ckey = (str(device), I, h, fp8, tuple(vals))
    hit = _table_cache.get(ckey)
    if hit is not None:
        return hit
    for i, r in enumerate(rows):
        if r[0].shape != gs or r[1].shape != gs or r[2].shape != ds or r[0].dtype != want or r[1].dtype != want or r[2].dtype != want:
            raise ValueError(f"experts[{i}]: weights must be {want} of shapes {gs}, {gs}, {ds}")
        if fp8 and (r[3] is None or r[4] is None or r[5] is None):
            raise ValueError("fp8 expert weights need their *_scale_inv block scales")
    if fp8:
        bi, bh = -(-I // 128), -(-h // 128)
        for i, r in enumerate(rows):
            if r[3].shape != (bi, bh) or r[4].shape != (bi, bh) or r[5].shape != (bh, bi) or r[3].dtype != torch.float32:
                raise ValueError(f"experts[{i}]: block scales must be fp32 of shapes {(bi, bh)}, {(bi, bh)}, {(bh, bi)}")
    t = _upload_words(vals, device)
    cols = [t[c * E:(c + 1) * E] for c in range(ncol)]
    out = ExpertPointers(E, h, I, fp8, cols[0], cols[1], cols[2], *(cols[3:] if fp8 else (None, None, None)))
    if len(_table_cache) >= _TABLE_CACHE_MAX:
        _table_cache.clear()
    _table_cache[ckey] = out       # (holds the device table only; the weights stay the engine's)
    return out


PHASE_GATE_UP, PHASE_DOWN, PHASE_BOTH = 1, 2, 3


def grouped_swiglu(x: torch.Tensor, row_map, ptrs: ExpertPointers, offsets: torch.Tensor, n_rows: int,
                   act: torch.Tensor | None = None, y: torch.Tensor | None = None, phases: int = PHASE_BOTH,
                   rows_bound: int | None = None, checked: bool = False, stream: int | None = None):
    """All experts' SwiGLU MLPs on their row ranges.  x: bf16 sorted rows [n_rows,h], or the
    unsorted matrix with row_map int32 [n_rows].  Returns y bf16 [n_rows,h] (sorted-row order).

    `ptrs` and `offsets` may describe a sub-range of a layer's experts (offsets = a slice
    offsets[a:b+1] of the layer's, absolute sorted rows): x, row_map, act and y stay the layer's
    full buffers, and rows_bound, if known, is the number of rows inside the range (it sizes the
    launch and picks the tile shape; default: n_rows).
    checked / stream: a caller that walks one layer in many waves passes the same x, row_map, act and y every
    time; it validates them on the first wave, says so, and passes the stream it looked up once."""
    h, I, E = ptrs.hidden, ptrs.inter, ptrs.n_experts
    if checked:
        if offsets.shape[0] != E + 1:
            raise ValueError(f"offsets must have {E + 1} entries, got {offsets.shape[0]}")
        if rows_bound is not None:
            n_rows = rows_bound
        st = _stream() if stream is None else stream
        fn = N.lib().moe_grouped_swiglu_w8a16 if ptrs.fp8 else N.lib().moe_grouped_swiglu_bf16
        scales = (_ptr(ptrs.s_gate), _ptr(ptrs.s_up), _ptr(ptrs.s_down)) if ptrs.fp8 else ()
        N.check(fn(x.data_ptr(), x.shape[0], _ptr(row_map), _ptr(ptrs.w_gate), _ptr(ptrs.w_up), _ptr(ptrs.w_down), *scales,
                   offsets.data_ptr(), n_rows, E, h, I, act.data_ptr(), y.data_ptr(), phases, None, 0, st), "moe_grouped_swiglu")
        return y
    _need(x, torch.bfloat16, "x")
    if x.shape[1] != h:
        raise ValueError(f"x has hidden size {x.shape[1]}, experts expect {h}")
    if row_map is None and x.shape[0] < n_rows:
        raise ValueError(f"x has {x.shape[0]} rows, need {n_rows}")
    if row_map is not None:
        _need(row_map, torch.int32, "row_map", (n_rows,))
    _need(offsets, torch.int32, "offsets", (E + 1,))
    dev = x.device
    if act is None:
        act = torch.empty((n_rows, I), dtype=torch.bfloat16, device=dev)
    if y is None:
        y = torch.empty((n_rows, h), dtype=torch.bfloat16, device=dev)
    _need(act, torch.bfloat16, "act", (n_rows, I))
    _need(y, torch.bfloat16, "y", (n_rows, h))
    L = N.lib()
    if rows_bound is not None:
        if not 0 <= rows_bound <= n_rows:
            raise ValueError(f"rows_bound {rows_bound} outside [0, {n_rows}]")
        n_rows = rows_bound
    if ptrs.fp8:
        N.check(L.moe_grouped_swiglu_w8a16(_ptr(x), x.shape[0], _ptr(row_map), _ptr(ptrs.w_gate), _ptr(ptrs.w_up),
                                           _ptr(ptrs.w_down), _ptr(ptrs.s_gate), _ptr(ptrs.s_up),
                                           _ptr(ptrs.s_down), _ptr(offsets), n_rows, E, h, I, _ptr(act), _ptr(y),
                                           phases, None, 0, _stream()), "moe_grouped_swiglu_w8a16")
    else:
        N.check(L.moe_grouped_swiglu_bf16(_ptr(x), x.shape[0], _ptr(row_map), _ptr(ptrs.w_gate), _ptr(ptrs.w_up),
                                          _ptr(ptrs.w_down), _ptr(offsets), n_rows, E, h, I, _ptr(act), _ptr(y),
                                          phases, None, 0, _stream()), "moe_grouped_swiglu_bf16")
    return y


def dequant_fp8_block128(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """bf16(f32(q) * scale[i//128, j//128]) -- deepseek_v3_dequantization (Wrapper.py:109-138)."""
    _need(q, torch.float8_e4m3fn, "q")
    rows, cols = q.shape
    _need(scale, torch.float32, "scale", (-(-rows // 128), -(-cols // 128)))
    out = torch.empty((rows, cols), dtype=torch.bfloat16, device=q.device)
    N.check(N.lib().moe_dequant_fp8_block128(_ptr(q), _ptr(scale), rows, cols, _ptr(out), _stream()),
            "moe_dequant_fp8_block128")
    return out


def combine(y: torch.Tensor, pos: torch.Tensor, topk_idx, topk_w: torch.Tensor, shared, mode: int,
            out: torch.Tensor | None = None, residual: torch.Tensor | None = None):
    """out[t] = sum_j w[t,j] * y[pos[t*k+j]] (+ shared[t]); y bf16 [n*k,h] in sorted-row order.
    residual: optional bf16 [n,h] added last (the decoder layer's `residual + hidden_states`,
    modeling_deepseek_v3.py:1365); `out` may be the residual buffer itself."""
    n, k = topk_w.shape
    h = y.shape[1]
    _need(y, torch.bfloat16, "y", (n * k, h))
    _need(pos, torch.int32, "pos", (n * k,))
    _need(topk_w, torch.float32, "topk_weight")
    if topk_idx is not None:
        _need(topk_idx, torch.int32, "topk_idx", (n, k))
    if shared is not None:
        _need(shared, torch.bfloat16, "shared", (n, h))
    if residual is not None:
        _need(residual, torch.bfloat16, "residual", (n, h))
    if out is None:
        out = torch.empty((n, h), dtype=torch.bfloat16, device=y.device)
    _need(out, torch.bfloat16, "out", (n, h))
    L = N.lib()
    if residual is None:
        N.check(L.moe_combine(_ptr(y), _ptr(pos), _ptr(topk_idx), _ptr(topk_w), _ptr(shared), n, k, h, mode,
                              _ptr(out), _stream()), "moe_combine")
    else:
        N.check(L.moe_combine_residual(_ptr(y), _ptr(pos), _ptr(topk_idx), _ptr(topk_w), _ptr(shared),
                                       _ptr(residual), n, k, h, mode, _ptr(out), _stream()), "moe_combine_residual")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, out: torch.Tensor | None = None):
    """post_attention_layernorm (DeepseekV3RMSNorm.forward, modeling_deepseek_v3.py:125-150):
    x bf16 [n,h], weight bf16 [h] -> bf16 [n,h]."""
    _need(x, torch.bfloat16, "x")
    n, h = x.shape
    _need(weight, torch.bfloat16, "weight", (h,))
    if out is None:
        out = torch.empty_like(x)
    _need(out, torch.bfloat16, "out", (n, h))
    N.check(N.lib().moe_rmsnorm(_ptr(x), _ptr(weight), float(eps), n, h, _ptr(out), _stream()), "moe_rmsnorm")
    return out
