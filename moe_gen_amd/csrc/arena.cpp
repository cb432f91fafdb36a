// Weight-arena index: the wire format that tells where each module's tensors lie inside one
// contiguous host arena.
//
// Replaces, for the MoE weights, the reference's
//   tensor_meta {offset, tensor_shape, byte_size}     core/Parameter_Server/Parameter_Server.h:48-59
//   compute_serialized_size / serialize_map_to_buffer core/Parameter_Server/posix_shm.cpp:167-268
//   deserialize_map_from_buffer                       core/Parameter_Server/posix_shm.cpp:270-357
//   Weights_Storage::Init (base + offset views)       core/Weights_Storage/Weights_Storage.cpp:52-77
// Format (native-endian, no padding):
//   u64 n_modules
//   per module:  u64 len, key bytes, u64 n_tensors
//     per tensor: u64 len, key bytes, i64 offset, i64 byte_size, u64 ndim, i64 shape[ndim]
// The reference walks unordered_maps, so the order of modules and tensors on the wire is
// unspecified there; here it is insertion order on writing and any order on reading.  A key
// that appears twice overwrites the earlier entry, as assignment into the reference's map does.
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace {

struct Tensor {
    std::string key;
    int64_t offset = 0, byte_size = 0;
    std::vector<int64_t> shape;
};

struct Module {
    std::string key;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, int> by_key;
};

}  // namespace

struct moe_arena_index {
    std::vector<Module> modules;
    std::unordered_map<std::string, int> by_key;
};

namespace {

Module& module_of(moe_arena_index* ix, const std::string& key) {
    auto it = ix->by_key.find(key);
    if (it != ix->by_key.end()) return ix->modules[it->second];
    ix->by_key[key] = (int)ix->modules.size();
    ix->modules.emplace_back();
    ix->modules.back().key = key;
    return ix->modules.back();
}

void put_tensor(Module& m, Tensor&& t) {
    auto it = m.by_key.find(t.key);
    if (it != m.by_key.end()) {
        m.tensors[it->second] = std::move(t);
        return;
    }
    m.by_key[t.key] = (int)m.tensors.size();
    m.tensors.push_back(std::move(t));
}

// bounded reader; the messages are the reference's (posix_shm.cpp:279-341)
struct Reader {
    const char* p;
    const char* end;
    bool take(void* dst, size_t n, const char* what) {
        if ((size_t)(end - p) < n) {
            moe::set_error("Buffer overflow (reading %s)", what);
            return false;
        }
        std::memcpy(dst, p, n);
        p += n;
        return true;
    }
    bool take_str(std::string& s, const char* what_len, const char* what_data) {
        uint64_t len;
        if (!take(&len, 8, what_len)) return false;
        if ((uint64_t)(end - p) < len) {
            moe::set_error("Buffer overflow (reading %s)", what_data);
            return false;
        }
        s.assign(p, (size_t)len);
        p += len;
        return true;
    }
};

size_t wire_size(const moe_arena_index* ix) {
    size_t total = 8;
    for (const Module& m : ix->modules) {
        total += 8 + m.key.size() + 8;
        for (const Tensor& t : m.tensors) total += 8 + t.key.size() + 16 + 8 + t.shape.size() * 8;
    }
    return total;
}

}  // namespace

extern "C" int moe_arena_index_create(moe_arena_index** out) {
    MOE_REQUIRE(out, "moe_arena_index_create: NULL argument");
    *out = new moe_arena_index();
    return MOE_OK;
}

extern "C" int moe_arena_index_destroy(moe_arena_index* ix) {
    delete ix;
    return MOE_OK;
}

extern "C" int moe_arena_index_add(moe_arena_index* ix, const char* module_key, const char* tensor_key,
                                   int64_t offset, int64_t byte_size, const int64_t* shape, int32_t ndim) {
    MOE_REQUIRE(ix && module_key && tensor_key, "moe_arena_index_add: NULL argument");
    MOE_REQUIRE(ndim >= 0 && ndim <= 8 && (shape || ndim == 0), "moe_arena_index_add: bad shape (ndim %d)", ndim);
    MOE_REQUIRE(offset >= 0 && byte_size >= 0, "moe_arena_index_add: negative offset %lld or size %lld",
                (long long)offset, (long long)byte_size);
    Tensor t;
    t.key = tensor_key;
    t.offset = offset;
    t.byte_size = byte_size;
    t.shape.assign(shape, shape + ndim);
    put_tensor(module_of(ix, module_key), std::move(t));
    return MOE_OK;
}

extern "C" int moe_arena_index_parse(const void* buf, size_t bytes, moe_arena_index** out) {
    MOE_REQUIRE(buf && out, "moe_arena_index_parse: NULL argument");
    Reader r{static_cast<const char*>(buf), static_cast<const char*>(buf) + bytes};
    moe_arena_index* ix = new moe_arena_index();
    auto fail = [&]() { delete ix; return MOE_ERR_INVALID; };
    uint64_t n_modules;
    if (!r.take(&n_modules, 8, "outer_size")) return fail();
    for (uint64_t i = 0; i < n_modules; ++i) {
        std::string mkey;
        if (!r.take_str(mkey, "outer key length", "outer key data")) return fail();
        uint64_t n_tensors;
        if (!r.take(&n_tensors, 8, "inner map size")) return fail();
        Module& m = module_of(ix, mkey);
        for (uint64_t j = 0; j < n_tensors; ++j) {
            Tensor t;
            if (!r.take_str(t.key, "inner key length", "inner key data")) return fail();
            int64_t pod[2];
            if (!r.take(pod, 16, "tensor_meta POD fields")) return fail();
            t.offset = pod[0];
            t.byte_size = pod[1];
            uint64_t ndim;
            if (!r.take(&ndim, 8, "tensor_shape size")) return fail();
            if (ndim > (uint64_t)(r.end - r.p) / 8) {
                moe::set_error("Buffer overflow (reading tensor_shape data)");
                return fail();
            }
            t.shape.resize((size_t)ndim);
            if (ndim && !r.take(t.shape.data(), (size_t)ndim * 8, "tensor_shape data")) return fail();
            put_tensor(m, std::move(t));
        }
    }
    *out = ix;
    return MOE_OK;
}

extern "C" size_t moe_arena_index_wire_size(const moe_arena_index* ix) { return ix ? wire_size(ix) : 0; }

extern "C" int moe_arena_index_serialize(const moe_arena_index* ix, void* buf, size_t capacity) {
    MOE_REQUIRE(ix && buf, "moe_arena_index_serialize: NULL argument");
    const size_t need = wire_size(ix);
    // the reference throws "Buffer overflow (...)" from inside the walk (posix_shm.cpp:204-266)
    MOE_REQUIRE(capacity >= need, "Buffer overflow (serialising %zu bytes into %zu)", need, capacity);
    char* p = static_cast<char*>(buf);
    auto put = [&](const void* src, size_t n) { std::memcpy(p, src, n); p += n; };
    auto put_u64 = [&](uint64_t v) { put(&v, 8); };
    put_u64(ix->modules.size());
    for (const Module& m : ix->modules) {
        put_u64(m.key.size());
        put(m.key.data(), m.key.size());
        put_u64(m.tensors.size());
        for (const Tensor& t : m.tensors) {
            put_u64(t.key.size());
            put(t.key.data(), t.key.size());
            put(&t.offset, 8);
            put(&t.byte_size, 8);
            put_u64(t.shape.size());
            if (!t.shape.empty()) put(t.shape.data(), t.shape.size() * 8);
        }
    }
    return MOE_OK;
}

extern "C" int32_t moe_arena_index_n_modules(const moe_arena_index* ix) { return ix ? (int32_t)ix->modules.size() : 0; }

extern "C" int moe_arena_index_module(const moe_arena_index* ix, int32_t i, const char** key, int32_t* n_tensors) {
    MOE_REQUIRE(ix && key && n_tensors, "moe_arena_index_module: NULL argument");
    MOE_REQUIRE(i >= 0 && i < (int)ix->modules.size(), "moe_arena_index_module: index %d outside [0,%zu)", i,
                ix->modules.size());
    *key = ix->modules[i].key.c_str();
    *n_tensors = (int32_t)ix->modules[i].tensors.size();
    return MOE_OK;
}

extern "C" int moe_arena_index_find(const moe_arena_index* ix, const char* module_key) {
    if (!ix || !module_key) return -1;
    auto it = ix->by_key.find(module_key);
    return it == ix->by_key.end() ? -1 : it->second;
}

extern "C" int moe_arena_index_tensor(const moe_arena_index* ix, int32_t i, int32_t j, const char** key, int64_t* offset,
                                      int64_t* byte_size, int32_t* ndim, const int64_t** shape) {
    MOE_REQUIRE(ix && key && offset && byte_size && ndim && shape, "moe_arena_index_tensor: NULL argument");
    MOE_REQUIRE(i >= 0 && i < (int)ix->modules.size(), "moe_arena_index_tensor: module %d outside [0,%zu)", i,
                ix->modules.size());
    const Module& m = ix->modules[i];
    MOE_REQUIRE(j >= 0 && j < (int)m.tensors.size(), "moe_arena_index_tensor: tensor %d outside [0,%zu)", j,
                m.tensors.size());
    const Tensor& t = m.tensors[j];
    *key = t.key.c_str();
    *offset = t.offset;
    *byte_size = t.byte_size;
    *ndim = (int32_t)t.shape.size();
    *shape = t.shape.data();
    return MOE_OK;
}

// Registers module `module_key` of the index with a stager: its tensors become copy sources at
// arena_base + offset (Weights_Storage::Init, Weights_Storage.cpp:69-76).  tensor_keys[i] goes to
// dst_offsets[i] of the slot; every listed tensor must exist and lie inside the arena.
static int add_module_from(moe_stager* st, int32_t type, const moe_arena_index* ix, const char* module_key,
                           const void* arena_base, size_t arena_bytes, int32_t n_tensors, const char* const* tensor_keys,
                           const size_t* dst_offsets, bool pageable) {
    MOE_REQUIRE(st && ix && module_key && arena_base && tensor_keys && dst_offsets,
                "moe_stage_add_module_from_arena / _segment: NULL argument");
    MOE_REQUIRE(n_tensors >= 1 && n_tensors <= 64, "moe_stage_add_module_from_arena: n_tensors %d outside [1,64]",
                n_tensors);
    auto it = ix->by_key.find(module_key);
    if (it == ix->by_key.end()) {
        moe::set_error("Module key not found in storage: %s", module_key);   // Weights_Storage.cpp:82-87
        return MOE_ERR_INVALID;
    }
    const Module& m = ix->modules[it->second];
    const void* src[64];
    size_t bytes[64];
    for (int i = 0; i < n_tensors; ++i) {
        auto jt = m.by_key.find(tensor_keys[i]);
        if (jt == m.by_key.end()) {
            moe::set_error("moe_stage_add_module_from_arena: module %s has no tensor %s", module_key, tensor_keys[i]);
            return MOE_ERR_INVALID;
        }
        const Tensor& t = m.tensors[jt->second];
        if (t.offset < 0 || t.byte_size < 0 || (uint64_t)t.offset + (uint64_t)t.byte_size > arena_bytes) {
            moe::set_error("moe_stage_add_module_from_arena: %s.%s (%lld bytes at offset %lld) lies outside the "
                           "%zu-byte arena", module_key, tensor_keys[i], (long long)t.byte_size, (long long)t.offset,
                           arena_bytes);
            return MOE_ERR_INVALID;
        }
        src[i] = static_cast<const char*>(arena_base) + t.offset;
        bytes[i] = (size_t)t.byte_size;
    }
    return pageable ? moe_stage_add_module_pageable(st, type, n_tensors, src, bytes, dst_offsets)
                    : moe_stage_add_module(st, type, n_tensors, src, bytes, dst_offsets);
}

extern "C" int moe_stage_add_module_from_arena(moe_stager* st, int32_t type, const moe_arena_index* ix,
                                               const char* module_key, const void* arena_base, size_t arena_bytes,
                                               int32_t n_tensors, const char* const* tensor_keys,
                                               const size_t* dst_offsets) {
    return add_module_from(st, type, ix, module_key, arena_base, arena_bytes, n_tensors, tensor_keys, dst_offsets, false);
}

// The same for a segment in ordinary (pageable) host memory, e.g. the reference's POSIX shm weight segment mapped
// into this process (posix_shm.cpp:36-92) without a second, pinned copy of the model: the module's copies go
// through the stager's bounce ring (moe_stage_set_bounce).
extern "C" int moe_stage_add_module_from_segment(moe_stager* st, int32_t type, const moe_arena_index* ix,
                                                 const char* module_key, const void* segment_base, size_t segment_bytes,
                                                 int32_t n_tensors, const char* const* tensor_keys,
                                                 const size_t* dst_offsets) {
    return add_module_from(st, type, ix, module_key, segment_base, segment_bytes, n_tensors, tensor_keys, dst_offsets, true);
}
