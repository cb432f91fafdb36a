"""Expert-weight staging with the verbs MoE-Gen's engine exposes to the model code
(core/MoE_Gen_Binding.cpp:45-65): get_weights, free_weights_buffer, clear_expert_buffer,
set_phase, reset_prefill_buffer, reset_weight_copy_queue.  The slot pool, the copy queue and all
of these verbs live in libmoe_mi355.so (moe_stage_*); this class maps module keys
("routed_expert_{L}_{e}", "shared_expert_{L}", Wrapper.py:457-468) to ids and tags and wraps slot
memory as torch tensors."""
from __future__ import annotations

import ctypes
import re

import torch

from . import _native as N

_ALIGN = 256
_KEY = re.compile(r"^(?:routed_expert_(\d+)_(\d+)|shared_expert_(\d+))$")


def _nbytes(shape, dtype) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n * torch.empty((), dtype=dtype).element_size()


class StagedExpert(torch.nn.Module):
    """An expert whose weights live in pinned host memory and reach the GPU through a Stager (or
    MoE-Gen's core_engine): the attribute surface of the reference's Expert_Wrapper
    (Wrapper.py:437-468) that block.staged_experts_forward consumes -- `.module`, `.core_engine`,
    `.get_weights`, `.expert_weights_idx`, `.layer_idx`, `.expert_idx`, `.weight_dequant_scale`."""

    def __init__(self, expert_module, layer_idx: int, expert_idx: int, core_engine, weight_dequant_scale=None):
        super().__init__()
        self.module = expert_module
        self.layer_idx, self.expert_idx = layer_idx, expert_idx
        self.core_engine = core_engine
        self.get_weights = True
        self.weight_dequant_scale = weight_dequant_scale
        self.expert_weights_idx = (f"routed_expert_{layer_idx}_{expert_idx}" if expert_idx >= 0
                                   else f"shared_expert_{layer_idx}")


class Stager:
    """module_shapes: {module_type: {tensor_name: (shape, dtype)}} -- the reference's
    GPU_Buffer_Config.module_shapes (deepseekv3_initializer.py:938-957);
    n_slots: {module_type: slots in the prefill phase}; n_slots_decoding: optional larger
    counts for the decoding phase (num_decoding_module_buffer, :918-927);
    backend "device": slots in HBM, sources must be pinned host tensors;
    backend "host": slots in host memory, plain memcpy (host-only tests);
    bounce_chunks > 0: a ring of that many pinned chunks of bounce_chunk_bytes through which modules
    whose sources lie in ordinary (pageable) memory are copied (Arena.stream_from,
    add_module(..., pageable=True)), bounce_threads host threads per chunk fill."""

    # free_weights_buffer records an event on the caller's stream and the next copy into the slot
    # waits for it: a caller need not drain its stream before letting go of weights (the
    # reference's pool flips a host flag, so its callers synchronise first, Wrapper.py:512-517)
    stream_ordered_release = True

    def __init__(self, module_shapes: dict, n_slots: dict, device="cuda", n_slots_decoding: dict | None = None,
                 model_type: str = "", num_hidden_layers: int = 0, num_local_experts: int = 0,
                 backend: str = "device", bounce_chunks: int = 0, bounce_chunk_bytes: int = 32 << 20,
                 bounce_threads: int = 8):
        self.backend = backend
        self.device = torch.device("cpu") if backend == "host" else torch.device(device)
        self.model_type = model_type
        self.num_hidden_layers = num_hidden_layers
        self.num_local_experts = num_local_experts
        self.types = list(module_shapes.keys())
        self.layout = {}       # type -> {name: (offset, bytes, shape, dtype)}
        self.pools = {}        # type -> uint8 tensor [n_total, slot_bytes]
        self.n_prefill = dict(n_slots)
        self.n_decoding = dict(n_slots_decoding or n_slots)
        slot_bytes, totals, mems = [], [], []
        for t in self.types:
            off, lay = 0, {}
            for name, (shape, dtype) in module_shapes[t].items():
                b = _nbytes(shape, dtype)
                lay[name] = (off, b, tuple(shape), dtype)
                off += -(-b // _ALIGN) * _ALIGN
            self.layout[t] = lay
            total = max(self.n_prefill[t], self.n_decoding.get(t, 0))
            self.pools[t] = torch.zeros((total, off), dtype=torch.uint8, device=self.device)
            slot_bytes.append(off)
            totals.append(total)
            mems.append(self.pools[t].data_ptr())
        nt = len(self.types)
        self._h = ctypes.c_void_p()
        N.check(N.lib().moe_stage_create(ctypes.byref(self._h), nt, (ctypes.c_size_t * nt)(*slot_bytes),
                                         (ctypes.c_int32 * nt)(*totals), (ctypes.c_void_p * nt)(*mems),
                                         1 if backend == "host" else 0), "moe_stage_create")
        N.check(N.lib().moe_stage_set_model(self._h, model_type.encode(), num_hidden_layers, num_local_experts),
                "moe_stage_set_model")
        for i, t in enumerate(self.types):
            N.check(N.lib().moe_stage_set_phase_slots(self._h, i, self.n_prefill[t],
                                                      max(self.n_prefill[t], self.n_decoding.get(t, 0))),
                    "moe_stage_set_phase_slots")
        self.bounce = False
        if bounce_chunks:
            self.set_bounce(bounce_chunks, bounce_chunk_bytes, bounce_threads)
        self.ids = {}          # module_key -> id
        self.type_of = {}      # module_key -> type
        self._src = []         # keeps the host tensors alive
        self.phase = "prefill"

    def _stream(self):
        return None if self.backend == "host" else torch.cuda.current_stream().cuda_stream

    def set_bounce(self, n_chunks: int = 8, chunk_bytes: int = 32 << 20, n_threads: int = 8) -> None:
        """Allocate the ring of pinned chunks that modules with pageable sources travel through."""
        N.check(N.lib().moe_stage_set_bounce(self._h, n_chunks, chunk_bytes, n_threads), "moe_stage_set_bounce")
        self.bounce = True

    def add_module(self, module_key: str, module_type: str, tensors: dict, pageable: bool = False) -> int:
        """Register one module (Weights_Storage's module_key -> tensor_key -> host buffer map,
        core/Weights_Storage/Weights_Storage.cpp:52-90) at the tail of its type's copy queue.
        pageable: the tensors lie in ordinary host memory and go through the bounce ring."""
        lay = self.layout[module_type]
        if set(tensors) != set(lay):
            raise RuntimeError(f"module {module_key}: tensors {sorted(tensors)} do not match the slot layout {sorted(lay)}")
        n = len(lay)
        src, nbytes, offs = [], [], []
        for name, (off, b, shape, dtype) in lay.items():
            t = tensors[name]
            if tuple(t.shape) != shape or t.dtype != dtype or not t.is_contiguous() or t.is_cuda:
                raise RuntimeError(f"module {module_key}.{name}: expected a contiguous host {dtype} tensor of shape {shape}")
            if self.backend == "device" and not pageable and not t.is_pinned():
                raise RuntimeError(f"module {module_key}.{name}: host tensor must be pinned (allocate with pin_memory=True), "
                                   "or registered with pageable=True on a stager with a bounce ring")
            src.append(t.data_ptr()); nbytes.append(b); offs.append(off)
            self._src.append(t)
        if pageable and not self.bounce:
            self.set_bounce()
        add = N.lib().moe_stage_add_module_pageable if pageable else N.lib().moe_stage_add_module
        mid = add(self._h, self.types.index(module_type), n, (ctypes.c_void_p * n)(*src),
                  (ctypes.c_size_t * n)(*nbytes), (ctypes.c_size_t * n)(*offs))
        if mid < 0:
            N.check(mid, "moe_stage_add_module")
        self._register(module_key, module_type, mid)
        return mid

    def _register(self, module_key: str, module_type: str, mid: int) -> None:
        self.ids[module_key] = mid
        self.type_of[module_key] = module_type
        m = _KEY.match(module_key)
        if m:        # the tag clear_expert_buffer selects by
            layer, expert = (int(m.group(1)), int(m.group(2))) if m.group(1) is not None else (int(m.group(3)), -1)
            N.check(N.lib().moe_stage_tag_module(self._h, mid, layer, expert), "moe_stage_tag_module")

    def add_module_from_arena(self, module_key: str, module_type: str, arena) -> int:
        """Register `module_key` with its tensors read in place from an Arena (the reference's
        Weights_Storage views into the shared weight segment, Weights_Storage.cpp:52-77)."""
        lay = self.layout[module_type]
        entries = arena.index.modules().get(module_key)
        if entries is None:
            raise RuntimeError(f"Module key not found in storage: {module_key}")
        for name, (off, b, shape, dtype) in lay.items():
            if name not in entries:
                raise RuntimeError(f"module {module_key}: arena has no tensor {name}")
            if entries[name][1] != b or tuple(entries[name][2]) != shape:
                raise RuntimeError(f"module {module_key}.{name}: arena entry {entries[name][1:]} does not match "
                                   f"the slot layout ({b} bytes, shape {shape})")
        pageable = bool(getattr(arena, "pageable", False))
        if self.backend == "device" and not pageable and not arena.data.is_pinned():
            raise RuntimeError("the arena must be pinned host memory (allocate it with pin_memory=True), or a "
                               "segment adopted with Arena.stream_from")
        if pageable and not self.bounce:
            self.set_bounce()
        n = len(lay)
        keys = (ctypes.c_char_p * n)(*[k.encode() for k in lay])
        offs = (ctypes.c_size_t * n)(*[v[0] for v in lay.values()])
        add = N.lib().moe_stage_add_module_from_segment if pageable else N.lib().moe_stage_add_module_from_arena
        mid = add(self._h, self.types.index(module_type), arena.index._h, module_key.encode(), arena.data.data_ptr(),
                  arena.data.numel(), n, keys, offs)
        if mid < 0:
            N.check(mid, "moe_stage_add_module_from_arena")
        self._src.append(arena)
        self._register(module_key, module_type, mid)
        return mid

    def pool_size(self, module_type: str) -> int:
        """Slots of `module_type` usable in the current phase (the rule the pools were sized by: a type
        without a decoding entry keeps its prefill slots, and the decoding pool never shrinks)."""
        n = self.n_prefill[module_type]
        return max(n, self.n_decoding.get(module_type, 0)) if self.phase == "decoding" else n

    def set_policy(self, module_type: str, policy: str) -> None:
        """"cyclic": every module of the type is copied in registration order whether or not it
        will be used (the reference's worker, HtoD_Engine.cpp:201-268); "on_demand": only the
        modules named by fetch() / get_weights() are copied."""
        if policy not in ("cyclic", "on_demand"):
            raise RuntimeError(f"unknown staging policy {policy!r}")
        N.check(N.lib().moe_stage_set_policy(self._h, self.types.index(module_type), 1 if policy == "on_demand" else 0),
                "moe_stage_set_policy")

    def fetch(self, module_keys) -> int:
        """Enqueue the copies of the listed modules that are not resident, in the given order;
        returns how many copies were issued."""
        ids = [self._id(k) for k in module_keys]
        n = len(ids)
        done = ctypes.c_int32(0)
        N.check(N.lib().moe_stage_fetch(self._h, (ctypes.c_int32 * max(n, 1))(*ids), n, ctypes.byref(done)),
                "moe_stage_fetch")
        return done.value

    def pump(self) -> int:
        r = N.lib().moe_stage_pump(self._h)
        if r < 0:
            N.check(r, "moe_stage_pump")
        return r

    def _id(self, module_key: str) -> int:
        if module_key not in self.ids:
            # the reference throws from Weights_Storage::get_module_weights_storage (:82-87)
            raise RuntimeError(f"Module key not found: {module_key}")
        return self.ids[module_key]

    def get_weights(self, module_key: str) -> dict:
        """Tensors aliasing the slot that holds `module_key`; the current stream is made to wait
        for the copy (GPU_Weight_Buffer::get_weights, GPU_Weight_Buffer.cpp:171-246, without the
        host-side wait)."""
        slot = ctypes.c_int32(-1)
        N.check(N.lib().moe_stage_acquire(self._h, self._id(module_key), self._stream(), ctypes.byref(slot)),
                "moe_stage_acquire")
        t = self.type_of[module_key]
        row = self.pools[t][slot.value]
        return {name: row[off:off + b].view(dtype).view(shape) for name, (off, b, shape, dtype) in self.layout[t].items()}

    def free_weights_buffer(self, module_key: str) -> None:
        N.check(N.lib().moe_stage_release(self._h, self._id(module_key), self._stream()), "moe_stage_release")

    def resident(self, module_key: str) -> bool:
        r = N.lib().moe_stage_resident(self._h, self._id(module_key))
        if r < 0:
            N.check(r, "moe_stage_resident")
        return bool(r)

    def clear_expert_buffer(self, layer_idx: int, expert_idx: int) -> int:
        """Release slots still held by routed experts that were prefetched but skipped (no tokens):
        experts < expert_idx of this layer and every expert of the previous MoE layer
        (GPU_Weight_Buffer::clear_expert_buffer, GPU_Weight_Buffer.cpp:261-308).  Returns how many."""
        r = N.lib().moe_stage_clear_expert_buffer(self._h, layer_idx, expert_idx, self._stream())
        if r < 0:
            N.check(r, "moe_stage_clear_expert_buffer")
        return r

    def set_phase(self, phase: str) -> None:
        """"decoding" grows the pools to their decoding size (MoE_Gen::set_phase -> resize_buffer,
        core/MoE_Gen.cpp:128-134, GPU_Weight_Buffer.cpp:103-142); "prefill" records the phase.  The
        engine follows "prefill" with reset_prefill_buffer() and reset_weight_copy_queue()
        (moe_gen/engine.py:680-683)."""
        N.check(N.lib().moe_stage_set_phase(self._h, str(phase).encode()), "moe_stage_set_phase")
        self.phase = phase

    def reset_prefill_buffer(self) -> None:
        """Pools back to their prefill size, residency dropped (GPU_Weight_Buffer.cpp:310-379)."""
        N.check(N.lib().moe_stage_reset_prefill_buffer(self._h), "moe_stage_reset_prefill_buffer")

    def reset_weight_copy_queue(self) -> None:
        """Cyclic queues back to registration order (HtoD_Engine.cpp:295-311)."""
        N.check(N.lib().moe_stage_reset_weight_copy_queue(self._h), "moe_stage_reset_weight_copy_queue")

    def stats(self):
        c, b = ctypes.c_int64(), ctypes.c_int64()
        N.check(N.lib().moe_stage_stats(self._h, ctypes.byref(c), ctypes.byref(b)), "moe_stage_stats")
        return c.value, b.value

    def sync(self) -> None:
        N.check(N.lib().moe_stage_sync(self._h), "moe_stage_sync")

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            N.lib().moe_stage_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
