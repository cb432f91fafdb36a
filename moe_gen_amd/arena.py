"""Weight arena: one contiguous pinned host buffer holding every module's tensors, plus the
index that says where each lies -- the reference's shared weight segment and its
module_key -> tensor_key -> {offset, shape, byte_size} map (Parameter_Server.h:48-59,
Weights_Storage.cpp:52-77), in the reference's wire format (posix_shm.cpp:167-357).

The reference maps a POSIX shm segment and registers it with the GPU runtime
(posix_shm.cpp allocate_shared_pinned_memory).  Registering existing memory is not supported
here, so an arena is either ALLOCATED pinned and filled by copy (`pack`, `from_bytes`: a second
copy of the weights in host memory), or left where it is, in ordinary memory, and streamed
through the stager's small ring of pinned chunks (`stream_from`: the host holds the model once)."""
from __future__ import annotations

import ctypes

import torch

from . import _native as N

_ALIGN = 256


class ArenaIndex:
    """module_key -> tensor_key -> (offset, byte_size, shape); parse/serialise in libmoe_mi355.so."""

    def __init__(self, handle=None):
        self._h = handle if handle is not None else ctypes.c_void_p()
        if handle is None:
            N.check(N.lib().moe_arena_index_create(ctypes.byref(self._h)), "moe_arena_index_create")

    @classmethod
    def parse(cls, data: bytes) -> "ArenaIndex":
        h = ctypes.c_void_p()
        buf = (ctypes.c_char * max(len(data), 1)).from_buffer_copy(data.ljust(1, b"\0"))
        N.check(N.lib().moe_arena_index_parse(ctypes.cast(buf, ctypes.c_void_p), len(data), ctypes.byref(h)),
                "moe_arena_index_parse")
        return cls(h)

    def add(self, module_key: str, tensor_key: str, offset: int, byte_size: int, shape) -> None:
        shape = [int(s) for s in shape]
        arr = (ctypes.c_int64 * max(len(shape), 1))(*shape)
        N.check(N.lib().moe_arena_index_add(self._h, module_key.encode(), tensor_key.encode(), offset, byte_size,
                                            arr, len(shape)), "moe_arena_index_add")

    def serialize(self) -> bytes:
        n = N.lib().moe_arena_index_wire_size(self._h)
        buf = ctypes.create_string_buffer(n)
        N.check(N.lib().moe_arena_index_serialize(self._h, ctypes.cast(buf, ctypes.c_void_p), n),
                "moe_arena_index_serialize")
        return buf.raw[:n]

    def modules(self) -> dict:
        """{module_key: {tensor_key: (offset, byte_size, shape tuple)}} in stored order."""
        L = N.lib()
        out = {}
        for i in range(L.moe_arena_index_n_modules(self._h)):
            key, nt = ctypes.c_char_p(), ctypes.c_int32()
            N.check(L.moe_arena_index_module(self._h, i, ctypes.byref(key), ctypes.byref(nt)), "moe_arena_index_module")
            tensors = {}
            for j in range(nt.value):
                tk, off, nb, nd = ctypes.c_char_p(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int32()
                shp = ctypes.POINTER(ctypes.c_int64)()
                N.check(L.moe_arena_index_tensor(self._h, i, j, ctypes.byref(tk), ctypes.byref(off), ctypes.byref(nb),
                                                 ctypes.byref(nd), ctypes.byref(shp)), "moe_arena_index_tensor")
                tensors[tk.value.decode()] = (off.value, nb.value, tuple(shp[d] for d in range(nd.value)))
            out[key.value.decode()] = tensors
        return out

    def __contains__(self, module_key: str) -> bool:
        return N.lib().moe_arena_index_find(self._h, module_key.encode()) >= 0

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            N.lib().moe_arena_index_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Arena:
    """A pinned host buffer + its index.  `pack` lays tensors out back to back (256-byte aligned);
    `from_bytes` adopts an index and a data blob produced elsewhere (another process, a file)."""

    def __init__(self, index: ArenaIndex, data: torch.Tensor, pageable: bool = False):
        if data.dtype != torch.uint8 or data.dim() != 1 or data.is_cuda or not data.is_contiguous():
            raise RuntimeError("arena data must be a contiguous 1-D uint8 host tensor")
        self.index, self.data, self.pageable = index, data, pageable

    @classmethod
    def stream_from(cls, index_bytes: bytes, segment) -> "Arena":
        """Adopt a weight segment WHERE IT LIES, in ordinary (pageable) host memory -- e.g. the
        reference's shm segment mapped into this process (Weights_Storage.cpp:52-78,
        posix_shm.cpp:36-92), as a uint8 tensor over the mapping (torch.from_numpy(np.memmap(...))
        or torch.frombuffer).  Nothing is copied here: a Stager built with a bounce ring moves each
        module through a few pinned chunks on its way to HBM, so the host holds the weights once
        (from_bytes holds them twice: ~640 GB more for the DeepSeek-R1 checkpoint)."""
        ix = ArenaIndex.parse(index_bytes)
        data = segment if isinstance(segment, torch.Tensor) else torch.frombuffer(segment, dtype=torch.uint8)
        return cls(ix, data.reshape(-1), pageable=True)

    @classmethod
    def pack(cls, modules: dict, pin: bool = True) -> "Arena":
        """modules: {module_key: {tensor_key: host tensor}}."""
        ix = ArenaIndex()
        total, plan = 0, []
        for mk, tensors in modules.items():
            for tk, t in tensors.items():
                if t.is_cuda or not t.is_contiguous():
                    raise RuntimeError(f"{mk}.{tk}: arena tensors must be contiguous host tensors")
                nb = t.numel() * t.element_size()
                plan.append((mk, tk, t, total, nb))
                total += -(-nb // _ALIGN) * _ALIGN
        data = torch.zeros(max(total, 1), dtype=torch.uint8, pin_memory=pin)
        for mk, tk, t, off, nb in plan:
            data[off:off + nb].copy_(t.reshape(-1).view(torch.uint8))
            ix.add(mk, tk, off, nb, t.shape)
        return cls(ix, data)

    @classmethod
    def from_bytes(cls, index_bytes: bytes, data, pin: bool = True) -> "Arena":
        """data: bytes-like or a uint8 host tensor (e.g. a memory-mapped weight segment); it is
        copied into freshly allocated pinned memory."""
        ix = ArenaIndex.parse(index_bytes)
        src = data if isinstance(data, torch.Tensor) else torch.frombuffer(bytearray(data), dtype=torch.uint8)
        buf = torch.empty(max(src.numel(), 1), dtype=torch.uint8, pin_memory=pin)
        buf[:src.numel()].copy_(src.reshape(-1))
        return cls(ix, buf[:src.numel()] if src.numel() else buf)

    def tensor(self, module_key: str, tensor_key: str, dtype: torch.dtype) -> torch.Tensor:
        off, nb, shape = self.index.modules()[module_key][tensor_key]
        if off < 0 or off + nb > self.data.numel():
            raise RuntimeError(f"{module_key}.{tensor_key} lies outside the arena")
        return self.data[off:off + nb].view(dtype).view(shape)
