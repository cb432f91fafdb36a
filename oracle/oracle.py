"""CPU oracle for the MoE-layer hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  It wraps ``libmoe_oracle.so`` (the scalar C
restatement in ``moe_oracle.c``) with numpy and adds the pieces that are library
routines on fp32 arrays (the expert MLP as ``numpy.matmul``) and a pure-Python
model of the weight-slot pool.

bf16 tensors travel as ``uint16`` numpy arrays (raw bits), fp8 as ``uint8``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")


def build(force: bool = False) -> str:
    """Compile moe_oracle.c with gcc (seconds).  Returns the library path."""
    src = os.path.join(_HERE, "moe_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libmoe_oracle.so"])
    return _LIB_PATH


class RouterParams(ctypes.Structure):
    _fields_ = [
        ("n_tokens", ctypes.c_int32), ("hidden", ctypes.c_int32),
        ("n_experts", ctypes.c_int32), ("top_k", ctypes.c_int32),
        ("n_group", ctypes.c_int32), ("topk_group", ctypes.c_int32),
        ("scoring", ctypes.c_int32), ("method", ctypes.c_int32),
        ("norm_topk_prob", ctypes.c_int32), ("scale_mode", ctypes.c_int32),
        ("logits_bf16", ctypes.c_int32), ("weights_bf16", ctypes.c_int32),
        ("norm_eps", ctypes.c_float), ("routed_scaling_factor", ctypes.c_float),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_bf16_to_f32.restype = ctypes.c_float
        _lib.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.orc_fp8_e4m3fn_to_f32.restype = ctypes.c_float
        _lib.orc_fp8_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        _lib.orc_f32_to_fp8_e4m3fn.restype = ctypes.c_uint8
        _lib.orc_f32_to_fp8_e4m3fn.argtypes = [ctypes.c_float]
        _lib.orc_expf.restype = ctypes.c_float
        _lib.orc_expf.argtypes = [ctypes.c_float]
        _lib.orc_sigmoidf.restype = ctypes.c_float
        _lib.orc_sigmoidf.argtypes = [ctypes.c_float]
        for name in ("orc_router", "orc_router_from_logits", "orc_dispatch", "orc_combine"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ----------------------------------------------------------------------------
# conversions
# ----------------------------------------------------------------------------

def f32_to_bf16(a) -> np.ndarray:
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_bf16_n(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def bf16_to_f32(a) -> np.ndarray:
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().orc_bf16_to_f32_n(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def round_bf16(a) -> np.ndarray:
    """fp32 -> bf16 (RNE) -> fp32."""
    return bf16_to_f32(f32_to_bf16(a))


def fp8_table() -> np.ndarray:
    """All 256 e4m3fn byte values decoded to fp32."""
    L = lib()
    return np.array([L.orc_fp8_e4m3fn_to_f32(i) for i in range(256)], np.float32)


def fp8_to_f32(q) -> np.ndarray:
    return fp8_table()[_c(q, np.uint8)]


def expf(a) -> np.ndarray:
    a = _c(a, np.float32)
    out = np.empty_like(a)
    lib().orc_expf_n(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def sigmoidf(a) -> np.ndarray:
    a = _c(a, np.float32)
    out = np.empty_like(a)
    lib().orc_sigmoidf_n(_p(a), _p(out), ctypes.c_int64(a.size))
    return out


def dequant_block(q, scale, block: int = 128) -> np.ndarray:
    """Wrapper.py:109-138: bf16(f32(q) * scale[i//128, j//128]); returns bf16 bits."""
    q = _c(q, np.uint8)
    scale = _c(scale, np.float32)
    rows, cols = q.shape
    assert scale.shape == (-(-rows // block), -(-cols // block))
    out = np.empty((rows, cols), np.uint16)
    lib().orc_dequant_block(_p(q), _p(scale), rows, cols, block, _p(out))
    return out


def quant_block(x, block: int = 128):
    """deepseekv3_initializer.py:191-205 per_block_cast_to_fp8 -> (q uint8, scale fp32)."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    q = np.empty((rows, cols), np.uint8)
    scale = np.empty((-(-rows // block), -(-cols // block)), np.float32)
    lib().orc_quant_block(_p(x), rows, cols, block, _p(q), _p(scale))
    return q, scale


# ----------------------------------------------------------------------------
# router
# ----------------------------------------------------------------------------

@dataclass
class RouterSpec:
    """Routing rules of one model family (field meanings as in moe_oracle.c)."""
    n_experts: int
    top_k: int
    scoring: str = "softmax"          # "softmax" | "sigmoid"
    method: str = "greedy"            # "greedy" | "group_limited_greedy" | "noaux_tc"
    n_group: int = 1
    topk_group: int = 1
    norm_topk_prob: bool = False
    scale_mode: int = 1               # 0 never, 1 when not normalised (V2), 2 always (V3)
    routed_scaling_factor: float = 1.0
    norm_eps: float = 1e-20
    logits_bf16: bool = False
    weights_bf16: bool = False

    @staticmethod
    def deepseek_v3(E, k, n_group, topk_group, norm=True, scale=2.5):
        return RouterSpec(E, k, "sigmoid", "noaux_tc", n_group, topk_group, norm, 2, scale)

    @staticmethod
    def deepseek_v2(E, k, method="greedy", n_group=1, topk_group=1, norm=False, scale=1.0):
        return RouterSpec(E, k, "softmax", method, n_group, topk_group, norm, 1, scale)

    @staticmethod
    def mixtral(E=8, k=2):
        return RouterSpec(E, k, "softmax", "greedy", 1, 1, True, 0, 1.0, 0.0, True, True)

    def params(self, n, h) -> RouterParams:
        return RouterParams(
            n, h, self.n_experts, self.top_k, self.n_group, self.topk_group,
            {"softmax": 0, "sigmoid": 1}[self.scoring],
            {"greedy": 0, "group_limited_greedy": 1, "noaux_tc": 2}[self.method],
            int(self.norm_topk_prob), self.scale_mode, int(self.logits_bf16),
            int(self.weights_bf16), self.norm_eps, self.routed_scaling_factor)


def logits(x_bf16, w_bf16) -> np.ndarray:
    x = _c(x_bf16, np.uint16)
    w = _c(w_bf16, np.uint16)
    n, h = x.shape
    E = w.shape[0]
    out = np.empty((n, E), np.float32)
    lib().orc_logits(_p(x), _p(w), n, h, E, _p(out))
    return out


def router(x_bf16, w_bf16, bias, spec: RouterSpec, want_scores=False):
    """-> (topk_idx int32 [n,k], topk_weight fp32 [n,k], logits fp32 [n,E][, scores])."""
    x = _c(x_bf16, np.uint16)
    w = _c(w_bf16, np.uint16)
    n, h = x.shape
    assert w.shape == (spec.n_experts, h)
    b = None if bias is None else _c(bias, np.float32)
    p = spec.params(n, h)
    idx = np.empty((n, spec.top_k), np.int32)
    wt = np.empty((n, spec.top_k), np.float32)
    lg = np.empty((n, spec.n_experts), np.float32)
    sc = np.empty((n, spec.n_experts), np.float32) if want_scores else None
    rc = lib().orc_router(_p(x), _p(w), _p(b), ctypes.byref(p), _p(idx), _p(wt), _p(lg), _p(sc))
    if rc:
        raise ValueError(f"orc_router rc={rc}")
    return (idx, wt, lg, sc) if want_scores else (idx, wt, lg)


def router_from_logits(lg, bias, spec: RouterSpec, want_scores=False):
    lg = _c(lg, np.float32)
    n, E = lg.shape
    assert E == spec.n_experts
    b = None if bias is None else _c(bias, np.float32)
    p = spec.params(n, 0)
    idx = np.empty((n, spec.top_k), np.int32)
    wt = np.empty((n, spec.top_k), np.float32)
    sc = np.empty((n, E), np.float32) if want_scores else None
    rc = lib().orc_router_from_logits(_p(lg), _p(b), ctypes.byref(p), _p(idx), _p(wt), _p(sc))
    if rc:
        raise ValueError(f"orc_router_from_logits rc={rc}")
    return (idx, wt, sc) if want_scores else (idx, wt)


# ----------------------------------------------------------------------------
# dispatch / combine
# ----------------------------------------------------------------------------

def dispatch(idx, n_experts):
    """-> counts [E], offsets [E+1], perm [n*k], pos [n*k] (all int32)."""
    idx = _c(idx, np.int32)
    n, k = idx.shape
    counts = np.empty(n_experts, np.int32)
    offsets = np.empty(n_experts + 1, np.int32)
    perm = np.empty(n * k, np.int32)
    pos = np.empty(n * k, np.int32)
    rc = lib().orc_dispatch(_p(idx), n, k, n_experts, _p(counts), _p(offsets), _p(perm), _p(pos))
    if rc:
        raise ValueError(f"orc_dispatch rc={rc}")
    return counts, offsets, perm, pos


def gather_rows(x_bf16, perm, k):
    x = _c(x_bf16, np.uint16)
    perm = _c(perm, np.int32)
    xs = np.empty((perm.size, x.shape[1]), np.uint16)
    lib().orc_gather_rows(_p(x), _p(perm), ctypes.c_int64(perm.size), k, x.shape[1], _p(xs))
    return xs


COMBINE_F32, COMBINE_BF16_PROD, COMBINE_BF16_SEQ = 0, 1, 2


def combine(ys_bf16, pos, idx, w, shared_bf16=None, mode=COMBINE_F32):
    ys = _c(ys_bf16, np.uint16)
    idx = _c(idx, np.int32)
    n, k = idx.shape
    h = ys.shape[1]
    pos = _c(pos, np.int32)
    w = _c(w, np.float32)
    sh = None if shared_bf16 is None else _c(shared_bf16, np.uint16)
    out = np.empty((n, h), np.uint16)
    rc = lib().orc_combine(_p(ys), _p(pos), _p(idx), _p(w), _p(sh), n, k, h, mode, _p(out))
    if rc:
        raise ValueError(f"orc_combine rc={rc}")
    return out


def rmsnorm(x_bf16, w_bf16, eps: float = 1e-6) -> np.ndarray:
    """post_attention_layernorm (modeling_deepseek_v3.py:125-150): bf16 [n,h] -> bf16 [n,h]."""
    x = _c(x_bf16, np.uint16)
    w = _c(w_bf16, np.uint16)
    n, h = x.shape
    if h % 8 or w.shape != (h,):
        raise ValueError("rmsnorm: hidden size must be a multiple of 8 and match the weight")
    out = np.empty((n, h), np.uint16)
    lib().orc_rmsnorm(_p(x), _p(w), ctypes.c_float(eps), n, h, _p(out))
    return out


def add_residual(a_bf16, residual_bf16) -> np.ndarray:
    """residual + hidden_states in bf16 (modeling_deepseek_v3.py:1365)."""
    a = _c(a_bf16, np.uint16)
    r = _c(residual_bf16, np.uint16)
    if a.shape != r.shape:
        raise ValueError("add_residual: shape mismatch")
    out = np.empty(a.shape, np.uint16)
    lib().orc_add_residual(_p(a), _p(r), ctypes.c_int64(a.size), _p(out))
    return out


# ----------------------------------------------------------------------------
# expert MLP and the whole layer
# ----------------------------------------------------------------------------

def silu(a):
    a = a.astype(np.float32)
    return a / (1.0 + np.exp(-a, dtype=np.float32))


def mlp_f32(x_f32, wg_f32, wu_f32, wd_f32):
    """down(silu(gate x) * up x) in fp32, no intermediate rounding
    (modeling_deepseek_v3.py:463-467 with every bf16(...) dropped)."""
    g = x_f32 @ wg_f32.T
    u = x_f32 @ wu_f32.T
    return (silu(g) * u) @ wd_f32.T


def mlp_ref_rounding(x_f32, wg_f32, wu_f32, wd_f32):
    """The same MLP with a bf16 rounding wherever torch's bf16 modules round:
    after each Linear, after SiLU, after the product (returns fp32 holding bf16 values)."""
    g = round_bf16(x_f32 @ wg_f32.T)
    u = round_bf16(x_f32 @ wu_f32.T)
    a = round_bf16(round_bf16(silu(g)) * u)
    return round_bf16(a @ wd_f32.T)


@dataclass
class LayerWeights:
    """fp32 views of the (bf16-valued) weights of one MoE layer."""
    gate: np.ndarray            # bf16 bits [E,h]
    bias: np.ndarray | None     # fp32 [E]
    wg: list                    # per expert fp32 [I,h]
    wu: list
    wd: list                    # per expert fp32 [h,I]
    shared: tuple | None = None  # (wg, wu, wd) fp32 with intermediate S*I


def layer(x_bf16, lw: LayerWeights, spec: RouterSpec, combine_mode=COMBINE_F32, rounding="f32"):
    """Whole MoE block on the CPU.

    rounding="f32": the fp32 evaluation of the reference math (bf16 only on inputs,
    weights and the final output) -- the reference for the 2e-2 bound; returns fp32.
    rounding="ref": rounds where the reference's bf16 modules round; returns bf16 bits.
    Returns (out, aux) with aux = dict(idx, w, counts, offsets, perm, pos).
    """
    x = _c(x_bf16, np.uint16)
    n, h = x.shape
    k = spec.top_k
    idx, w, lg = router(x, lw.gate, lw.bias, spec)
    counts, offsets, perm, pos = dispatch(idx, spec.n_experts)
    xf = bf16_to_f32(x)
    xs = xf[perm // k]
    mlp = mlp_f32 if rounding == "f32" else mlp_ref_rounding
    ys = np.zeros((n * k, h), np.float32)
    for e in range(spec.n_experts):
        a, b = offsets[e], offsets[e + 1]
        if b > a:
            ys[a:b] = mlp(xs[a:b], lw.wg[e], lw.wu[e], lw.wd[e])
    sh = None
    if lw.shared is not None:
        sh = mlp(xf, *lw.shared)
    aux = dict(idx=idx, w=w, logits=lg, counts=counts, offsets=offsets, perm=perm, pos=pos)
    if rounding == "f32":
        out = (ys[pos.reshape(n, k)] * w[:, :, None]).sum(axis=1, dtype=np.float32)
        if sh is not None:
            out = out + sh
        return out, aux
    out = combine(f32_to_bf16(ys), pos, idx, w, None if sh is None else f32_to_bf16(sh), combine_mode)
    return out, aux


# ----------------------------------------------------------------------------
# weight-slot pool model (GPU_Weight_Buffer.cpp:146-308, HtoD_Engine.cpp:201-268)
# ----------------------------------------------------------------------------

class SlotPoolModel:
    """Pure-Python model of the reference's slot pool and cyclic copy queue.

    One FIFO of module names per module type; `pump()` is one turn of the copy
    worker: for each type, if a slot is empty, pop the next name, copy it into
    the slot, mark it resident and push the name back (HtoD_Engine.cpp:201-268).
    `release` frees the slot of a resident module (GPU_Weight_Buffer.cpp:163-169);
    `clear_expert_buffer(L, e)` releases routed experts `< e` of layer L and every
    routed expert of the previous MoE layer, where "previous" wraps to the last
    layer for the first MoE layer(s) (GPU_Weight_Buffer.cpp:261-308).
    """

    def __init__(self, n_slots: dict, queues: dict, model_type: str, num_hidden_layers: int,
                 num_local_experts: int):
        self.slots = {t: [None] * n for t, n in n_slots.items()}
        self.queues = {t: list(names) for t, names in queues.items()}
        self.resident = {}
        self.model_type = model_type
        self.L = num_hidden_layers
        self.E = num_local_experts
        self.copies = []
        self.on_demand = set()      # module types taken out of the cyclic queue

    def fetch(self, names):
        """On-demand staging (not in the reference, whose worker copies every module): copy
        the listed modules that are not resident into the first empty slot of their type, in
        the given order."""
        type_of = {n: t for t, q in self.queues.items() for n in q}
        done = 0
        for name in names:
            if name in self.resident:
                continue
            t = type_of[name]
            if None not in self.slots[t]:
                raise RuntimeError(f"no free slot of type {t} for {name}")
            s = self.slots[t].index(None)
            self.slots[t][s] = name
            self.resident[name] = (t, s)
            self.copies.append((name, t, s))
            done += 1
        return done

    def pump(self):
        did = False
        for t in self.queues:
            if t in self.on_demand:
                continue
            if None in self.slots[t] and self.queues[t]:
                s = self.slots[t].index(None)
                name = self.queues[t].pop(0)
                self.slots[t][s] = name
                self.resident[name] = (t, s)
                self.queues[t].append(name)
                self.copies.append((name, t, s))
                did = True
        return did

    def release(self, name):
        t, s = self.resident.pop(name)
        self.slots[t][s] = None

    def prev_layer(self, layer_idx):
        if self.model_type == "deepseek_v2" and layer_idx in (0, 1):
            return self.L - 1
        if self.model_type == "deepseek_v3" and 0 <= layer_idx <= 3:
            return self.L - 1
        return layer_idx - 1

    def clear_expert_buffer(self, layer_idx, expert_idx):
        for e in range(expert_idx):
            name = f"routed_expert_{layer_idx}_{e}"
            if name in self.resident:
                self.release(name)
        pl = self.prev_layer(layer_idx)
        for e in range(self.E):
            name = f"routed_expert_{pl}_{e}"
            if name in self.resident:
                self.release(name)
