"""TEST INFRASTRUCTURE -- CPU restatement of the reference's weight-arena index wire format.

Follows core/Parameter_Server/posix_shm.cpp: compute_serialized_size (:167-190),
serialize_map_to_buffer (:196-268), deserialize_map_from_buffer (:270-357); tensor_meta is
{offset, tensor_shape, byte_size} (Parameter_Server.h:48-59).  size_t and int64_t are 8 bytes,
native (little) endian, nothing is padded.  The reference iterates unordered_maps, so the
order of entries on the wire is unspecified; this restatement writes dict order.

Only tests may import this module."""
import struct


def serialized_size(m: dict) -> int:
    total = 8
    for mk, inner in m.items():
        total += 8 + len(mk.encode()) + 8
        for tk, (offset, byte_size, shape) in inner.items():
            total += 8 + len(tk.encode()) + 16 + 8 + 8 * len(shape)
    return total


def serialize(m: dict) -> bytes:
    """m: {module_key: {tensor_key: (offset, byte_size, shape)}}"""
    out = [struct.pack("<Q", len(m))]
    for mk, inner in m.items():
        k = mk.encode()
        out += [struct.pack("<Q", len(k)), k, struct.pack("<Q", len(inner))]
        for tk, (offset, byte_size, shape) in inner.items():
            t = tk.encode()
            out += [struct.pack("<Q", len(t)), t, struct.pack("<qq", offset, byte_size), struct.pack("<Q", len(shape))]
            out += [struct.pack("<q", s) for s in shape]
    return b"".join(out)


def deserialize(buf: bytes) -> dict:
    pos = 0

    def take(n, what):
        nonlocal pos
        if pos + n > len(buf):
            raise RuntimeError(f"Buffer overflow (reading {what})")
        b = buf[pos:pos + n]
        pos += n
        return b

    m = {}
    (outer,) = struct.unpack("<Q", take(8, "outer_size"))
    for _ in range(outer):
        (kl,) = struct.unpack("<Q", take(8, "outer key length"))
        mk = take(kl, "outer key data").decode()
        (inner_n,) = struct.unpack("<Q", take(8, "inner map size"))
        inner = m.setdefault(mk, {})
        for _ in range(inner_n):
            (tl,) = struct.unpack("<Q", take(8, "inner key length"))
            tk = take(tl, "inner key data").decode()
            offset, byte_size = struct.unpack("<qq", take(16, "tensor_meta POD fields"))
            (nd,) = struct.unpack("<Q", take(8, "tensor_shape size"))
            if nd > (len(buf) - pos) // 8:
                raise RuntimeError("Buffer overflow (reading tensor_shape data)")
            shape = struct.unpack(f"<{nd}q", take(8 * nd, "tensor_shape data")) if nd else ()
            inner[tk] = (offset, byte_size, tuple(shape))
    return m
