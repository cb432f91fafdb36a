// Expert-weight staging: a pool of HBM slots per module type, filled from pinned host
// memory on a private copy stream in a fixed cyclic order, handed to the compute stream
// by events.
//
// Replaces, for weights, the reference's copy worker and slot pool:
//   HtoD_Engine::HtoD_Worker           core/HtoD_Engine/HtoD_Engine.cpp:201-268
//   HtoD_Engine::blocking_copy_        core/HtoD_Engine/HtoD_Engine.cpp:112-118
//   GPU_Weight_Buffer::acquireEmptyBuffer / releaseBuffer / get_weights /
//     weights_copy_complete            core/GPU_Weight_Buffer/GPU_Weight_Buffer.cpp:146-259
//   GPU_Weight_Buffer::resize_buffer / reset_prefill_buffer   :103-142, :310-379
//   HtoD_Engine::reset_weight_copy_queue                      HtoD_Engine.cpp:284-311
// The reference runs a host thread that copies one tensor at a time and synchronises
// the stream after each, then wakes the consumer through a condition variable.  Here
// no host thread exists and the host never waits: a copy is enqueued as soon as a slot
// is free (pump), the consumer's stream waits on the copy's event (acquire), and the
// next copy into a slot waits on the event recorded by the consumer when it let go of
// the slot (release).  The default copy order is the reference's: per type, the modules in
// the order they were registered, cyclically, whether or not the router will use them.
// A type can instead be switched to on-demand: nothing is copied until the caller names the
// modules it needs (fetch), typically the experts with a non-zero token count, busiest first.
//
// The reference's remaining verbs on the pool are here too, by module tag instead of by name:
//   GPU_Weight_Buffer::clear_expert_buffer    GPU_Weight_Buffer.cpp:261-308  (moe_stage_clear_expert_buffer)
//   MoE_Gen::set_phase -> resize_buffer       MoE_Gen.cpp:128-134            (moe_stage_set_phase)
//   MoE_Gen::reset_prefill_buffer / reset_weight_copy_queue   MoE_Gen.cpp:205-211
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "common.h"

namespace {

struct Piece {
    const void* src;
    size_t bytes, dst_off;
};

struct Module {
    int type = 0;
    std::vector<Piece> pieces;
    int slot = -1;               // -1: not resident
    bool held = false;           // acquired by a consumer and not yet released
    bool wanted = false;         // named by a fetch and not yet released (on-demand staging)
    int layer = -1, expert = -2; // tag: routed expert `expert` (>= 0) or shared expert (-1) of `layer`; -2 untagged
    hipEvent_t ready = nullptr;  // copy finished (device backend)
    bool pageable = false;       // sources are ordinary host memory: copies go through the pinned bounce ring
    uint64_t job_seq = 0;        // sequence number of this module's latest bounce job
};

struct Type {
    size_t slot_bytes = 0;
    int n_total = 0, n_active = 0;
    uint8_t* mem = nullptr;
    std::vector<int> owner;             // slot -> module id, -1 free
    // Hand-back of a slot (device backend).  A release only notes the consumer's stream (freed_pending); the next
    // copy that wants any such slot records ONE event per stream for all slots released since, and each of them then
    // refers to that event (freed_ev) under a ticket that grows with every record.
    std::vector<hipEvent_t> freed;      // one event object per slot
    std::vector<char> freed_pending;    // released, no event recorded yet
    std::vector<hipStream_t> freed_strm;
    std::vector<hipEvent_t> freed_ev;   // the event the next copy into the slot waits for (some slot's object)
    std::vector<uint64_t> freed_ticket;
    std::vector<char> freed_valid;
    std::vector<int> order;             // registration order
    std::deque<int> fifo;               // cyclic copy queue
    int policy = MOE_STAGE_CYCLIC;
    int n_prefill = 0, n_decoding = 0;  // slots per phase (0: the phase verbs leave this type alone)
};

// Copies out of PAGEABLE host memory (a mapped weight segment that was not allocated pinned): a worker thread
// moves each module through a ring of pinned chunks -- host memcpy into the next chunk (split over a few helper
// threads), then hipMemcpyAsync out of it on the copy stream -- so the segment is never copied whole and the
// pinned memory is n_chunks x chunk_bytes.  A chunk is refilled once the event recorded behind its last
// hipMemcpyAsync has completed; the memcpy into one chunk overlaps the DMA out of the others.
struct BounceJob {
    uint64_t seq = 0;
    uint8_t* dst = nullptr;
    std::vector<Piece> pieces;
    hipEvent_t wait_for = nullptr;   // release event of the slot's previous user (device backend), or null
    hipEvent_t ready = nullptr;
};

struct Bounce {
    int n_chunks = 0, n_threads = 1, device = 0, backend = MOE_STAGE_DEVICE;
    size_t chunk_bytes = 0;
    hipStream_t stream = nullptr;
    std::vector<uint8_t*> chunk;
    std::vector<hipEvent_t> done;
    std::vector<char> busy;
    int next = 0;
    std::thread worker;
    std::mutex mu;
    std::condition_variable cv_job, cv_done;
    std::deque<BounceJob> jobs;
    uint64_t enqueued = 0, issued = 0;   // jobs handed in / jobs whose copies have all been enqueued on the stream
    bool stop = false;
    int err = MOE_OK;
    std::string err_msg;

    void copy_in(uint8_t* dst, const uint8_t* src, size_t n) {   // pageable -> pinned, on n_threads threads
        const size_t min_part = 1u << 20;
        int parts = (int)std::min<size_t>((size_t)n_threads, (n + min_part - 1) / min_part);
        if (parts <= 1) { std::memcpy(dst, src, n); return; }
        std::vector<std::thread> th;
        const size_t per = ((n / parts) + 4095) & ~(size_t)4095;
        for (int i = 1; i < parts; ++i) {
            const size_t a = std::min(n, per * i), b = std::min(n, per * (i + 1));
            if (b > a) th.emplace_back([=] { std::memcpy(dst + a, src + a, b - a); });
        }
        std::memcpy(dst, src, std::min(n, per));
        for (auto& t : th) t.join();
    }
    int run_job(const BounceJob& j) {
        const bool dev = backend == MOE_STAGE_DEVICE;
        if (dev && j.wait_for) MOE_HIP_CHECK(hipStreamWaitEvent(stream, j.wait_for, 0));
        for (const Piece& p : j.pieces)
            for (size_t off = 0; off < p.bytes; off += chunk_bytes) {
                const size_t len = std::min(chunk_bytes, p.bytes - off);
                const int c = next;
                next = (next + 1) % n_chunks;
                if (dev && busy[c]) MOE_HIP_CHECK(hipEventSynchronize(done[c]));
                copy_in(chunk[c], static_cast<const uint8_t*>(p.src) + off, len);
                if (dev) {
                    MOE_HIP_CHECK(hipMemcpyAsync(j.dst + p.dst_off + off, chunk[c], len, hipMemcpyHostToDevice, stream));
                    MOE_HIP_CHECK(hipEventRecord(done[c], stream));
                    busy[c] = 1;
                } else {
                    std::memcpy(j.dst + p.dst_off + off, chunk[c], len);
                }
            }
        if (dev) MOE_HIP_CHECK(hipEventRecord(j.ready, stream));
        return MOE_OK;
    }
    void loop() {
        if (backend == MOE_STAGE_DEVICE) (void)hipSetDevice(device);
        for (;;) {
            BounceJob j;
            {
                std::unique_lock<std::mutex> lk(mu);
                cv_job.wait(lk, [&] { return stop || !jobs.empty(); });
                if (jobs.empty()) return;
                j = std::move(jobs.front());
                jobs.pop_front();
            }
            const int rc = run_job(j);
            {
                std::lock_guard<std::mutex> lk(mu);
                if (rc != MOE_OK && err == MOE_OK) { err = rc; err_msg = moe_last_error(); }
                issued = j.seq;
            }
            cv_done.notify_all();
        }
    }
    // blocks until the copies of job `seq` have been enqueued on the copy stream
    int wait_issued(uint64_t seq) {
        std::unique_lock<std::mutex> lk(mu);
        cv_done.wait(lk, [&] { return issued >= seq; });
        if (err != MOE_OK) { moe::set_error("bounce copy worker: %s", err_msg.c_str()); return err; }
        return MOE_OK;
    }
    void shutdown() {
        if (worker.joinable()) {
            { std::lock_guard<std::mutex> lk(mu); stop = true; }
            cv_job.notify_all();
            worker.join();
        }
        for (size_t i = 0; i < chunk.size(); ++i) {
            if (backend == MOE_STAGE_DEVICE) { if (chunk[i]) (void)hipHostFree(chunk[i]); if (done[i]) (void)hipEventDestroy(done[i]); }
            else std::free(chunk[i]);
        }
        chunk.clear(); done.clear(); busy.clear();
        n_chunks = 0;
    }
};

}  // namespace

struct moe_stager {
    int backend = MOE_STAGE_DEVICE;
    Bounce bounce;
    hipStream_t copy_stream = nullptr;
    std::vector<Type> types;
    std::vector<Module> modules;
    int64_t n_copies = 0, n_bytes = 0;
    int wrap_layers = 0;         // layers [0, wrap_layers) take the last layer as their "previous" one
    int num_hidden_layers = 0, num_local_experts = 0;
    int decoding = 0;
    int n_held = 0;              // modules acquired and not yet released
    // Events of one consumer stream are recorded in ticket order, so a wait for ticket T covers every smaller one.
    // Which ticket the copy stream already waits for, per consumer stream: for copies enqueued by the caller's
    // thread, and for the bounce worker's jobs (enqueued later, in job order).
    uint64_t ticket = 0;
    std::vector<std::pair<hipStream_t, uint64_t>> waited_direct, waited_jobs;
    std::mutex mu;
};

namespace {

int find_free(const Type& t) {
    for (int s = 0; s < t.n_active; ++s)
        if (t.owner[s] < 0) return s;
    return -1;
}

// One event per consumer stream for every slot released since the last call.  A wait that is still pending when a
// copy is enqueued costs the copy stream about 0.2 ms on this runtime: a wave of ten experts released one by one and
// refilled one by one, each behind its own event, lost 2.3 ms per wave (272 instead of 211 ms per DeepSeek-V3 layer
// once the host no longer waited for the GPU between waves); with one event per batch of releases the first copy
// waits and the others are covered by it.
int flush_released(moe_stager* st) {
    for (;;) {
        hipStream_t strm = nullptr;
        hipEvent_t ev = nullptr;
        for (Type& t : st->types)
            for (int s = 0; s < t.n_total; ++s) {
                if (!t.freed_pending[s]) continue;
                if (!ev) {
                    strm = t.freed_strm[s];
                    ev = t.freed[s];
                    MOE_HIP_CHECK(hipEventRecord(ev, strm));
                    ++st->ticket;
                } else if (t.freed_strm[s] != strm) {
                    continue;                 // another consumer stream: the next round
                }
                t.freed_pending[s] = 0;
                t.freed_ev[s] = ev;
                t.freed_ticket[s] = st->ticket;
                t.freed_valid[s] = 1;
            }
        if (!ev) return MOE_OK;
    }
}

// whether a wait for `ticket` of consumer stream `strm` is still needed; notes it as issued
bool need_wait(std::vector<std::pair<hipStream_t, uint64_t>>& waited, hipStream_t strm, uint64_t ticket) {
    for (auto& w : waited)
        if (w.first == strm) {
            if (w.second >= ticket) return false;
            w.second = ticket;
            return true;
        }
    waited.emplace_back(strm, ticket);
    return true;
}

// enqueue the copy of module `id` into free slot `slot` of its type
int copy_into(moe_stager* st, int id, int slot) {
    Module& m = st->modules[id];
    Type& t = st->types[m.type];
    uint8_t* dst = t.mem + (size_t)slot * t.slot_bytes;
    if (st->backend == MOE_STAGE_DEVICE && t.freed_pending[slot]) {
        int rc = flush_released(st);
        if (rc != MOE_OK) return rc;
    }
    if (m.pageable) {
        Bounce& b = st->bounce;
        if (b.n_chunks == 0) {
            moe::set_error("module %d has pageable sources but no bounce ring is configured (moe_stage_set_bounce)", id);
            return MOE_ERR_STATE;
        }
        BounceJob j;
        j.dst = dst;
        j.pieces = m.pieces;
        j.ready = m.ready;
        if (st->backend == MOE_STAGE_DEVICE && t.freed_valid[slot]) {
            if (need_wait(st->waited_jobs, t.freed_strm[slot], t.freed_ticket[slot])) j.wait_for = t.freed_ev[slot];
            t.freed_valid[slot] = 0;
        }
        {
            std::lock_guard<std::mutex> lk(b.mu);
            j.seq = ++b.enqueued;
            m.job_seq = j.seq;
            b.jobs.push_back(std::move(j));
        }
        b.cv_job.notify_one();
    } else if (st->backend == MOE_STAGE_DEVICE) {
        if (t.freed_valid[slot]) {
            if (need_wait(st->waited_direct, t.freed_strm[slot], t.freed_ticket[slot]))
                MOE_HIP_CHECK(hipStreamWaitEvent(st->copy_stream, t.freed_ev[slot], 0));
            t.freed_valid[slot] = 0;
        }
        for (const Piece& p : m.pieces)
            MOE_HIP_CHECK(hipMemcpyAsync(dst + p.dst_off, p.src, p.bytes, hipMemcpyHostToDevice, st->copy_stream));
        MOE_HIP_CHECK(hipEventRecord(m.ready, st->copy_stream));
    } else {
        for (const Piece& p : m.pieces) std::memcpy(dst + p.dst_off, p.src, p.bytes);
    }
    for (const Piece& p : m.pieces) st->n_bytes += (int64_t)p.bytes;
    st->n_copies += 1;
    t.owner[slot] = id;
    m.slot = slot;
    return MOE_OK;
}

// one turn of the copy worker for one type; returns 1 if a copy was enqueued, 0 if not, <0 on error
int pump_type(moe_stager* st, int ti) {
    Type& t = st->types[ti];
    if (t.policy != MOE_STAGE_CYCLIC || t.fifo.empty()) return 0;
    const int slot = find_free(t);
    if (slot < 0) return 0;
    // The next module in line that is not resident.  In the reference's order of use (modules
    // released in the order they were copied) the head of the queue never is; if the caller let go
    // of a later module first, resident ones keep their place in the cycle (they move to the back,
    // as after a copy) instead of blocking the free slot -- the reference would copy the head a
    // second time into the free slot (HtoD_Engine.cpp:201-268), which only costs bandwidth.
    size_t turns = 0;
    while (turns < t.fifo.size() && st->modules[t.fifo.front()].slot >= 0) {
        t.fifo.push_back(t.fifo.front());
        t.fifo.pop_front();
        ++turns;
    }
    if (turns == t.fifo.size()) return 0;     // every module of the type is resident
    const int id = t.fifo.front();
    t.fifo.pop_front();
    int rc = copy_into(st, id, slot);
    if (rc != MOE_OK) {
        t.fifo.push_front(id);   // not copied: it keeps its turn
        return rc;
    }
    t.fifo.push_back(id);  // the reference pushes the name back for the next pass
    return 1;
}

// on-demand copy of one module; 1 if enqueued, 0 if already resident, <0 on error
int fetch_one(moe_stager* st, int id) {
    Module& m = st->modules[id];
    if (m.slot >= 0) {
        m.wanted = true;
        return 0;
    }
    Type& t = st->types[m.type];
    int slot = find_free(t);
    if (slot < 0) {
        // A slot whose module nobody has acquired and no fetch has named -- left there by the cyclic prefetch before
        // the type was switched to on-demand, or by an earlier call's surplus -- is taken over: no consumer reads
        // it, and the new copy follows the old one on the copy stream.
        for (int s = 0; s < t.n_active && slot < 0; ++s) {
            Module& o = st->modules[t.owner[s]];
            if (!o.held && !o.wanted) {
                o.slot = -1;
                t.owner[s] = -1;
                slot = s;
            }
        }
    }
    if (slot < 0) {
        moe::set_error("moe_stage_fetch: no free slot of type %d for module %d (%d active slots, all held or named by "
                       "an earlier fetch)", m.type, id, t.n_active);
        return MOE_ERR_STATE;
    }
    int rc = copy_into(st, id, slot);
    if (rc != MOE_OK) return rc;
    m.wanted = true;
    return 1;
}

// hand the slot of a resident module back; the next copy into it waits for `stream`
int release_one(moe_stager* st, int id, hipStream_t stream) {
    Module& m = st->modules[id];
    Type& t = st->types[m.type];
    if (st->backend == MOE_STAGE_DEVICE) {
        t.freed_pending[m.slot] = 1;
        t.freed_strm[m.slot] = stream;
        t.freed_valid[m.slot] = 0;
    }
    t.owner[m.slot] = -1;
    m.slot = -1;
    if (m.held) --st->n_held;
    m.held = false;
    m.wanted = false;
    return MOE_OK;
}

// drop residency of every module of a type and rewind nothing: all its slots become free.  Refused
// while a consumer holds one of them (its kernels may still be queued and no event covers them).
int drop_residency(moe_stager* st, int ti, const char* who) {
    Type& t = st->types[ti];
    for (int s = 0; s < t.n_total; ++s)
        if (t.owner[s] >= 0 && st->modules[t.owner[s]].held) {
            moe::set_error("%s: module %d of type %d is still held (release it first)", who, t.owner[s], ti);
            return MOE_ERR_STATE;
        }
    if (st->bounce.n_chunks > 0) {
        int rc = st->bounce.wait_issued(st->bounce.enqueued);
        if (rc != MOE_OK) return rc;
    }
    if (st->backend == MOE_STAGE_DEVICE) {
        int rc = flush_released(st);        // (the consumers' streams are named now, while they certainly exist)
        if (rc != MOE_OK) return rc;
        MOE_HIP_CHECK(hipStreamSynchronize(st->copy_stream));
    }
    for (int s = 0; s < t.n_total; ++s) {
        if (t.owner[s] >= 0) {
            st->modules[t.owner[s]].slot = -1;
            st->modules[t.owner[s]].wanted = false;
        }
        t.owner[s] = -1;
    }
    return MOE_OK;
}

int pump_all(moe_stager* st) {
    int n = 0;
    for (size_t ti = 0; ti < st->types.size(); ++ti) {
        for (;;) {
            int r = pump_type(st, (int)ti);
            if (r < 0) return r;
            if (r == 0) break;
            ++n;
        }
    }
    return n;
}

}  // namespace

extern "C" int moe_stage_create(moe_stager** out, int32_t n_types, const size_t* slot_bytes, const int32_t* n_slots,
                                void* const* slot_mem, int32_t backend) {
    MOE_REQUIRE(out && slot_bytes && n_slots && slot_mem, "moe_stage_create: NULL argument");
    MOE_REQUIRE(n_types >= 1 && n_types <= 64, "moe_stage_create: n_types %d outside [1,64]", n_types);
    MOE_REQUIRE(backend == MOE_STAGE_DEVICE || backend == MOE_STAGE_HOST_MEMCPY, "moe_stage_create: bad backend %d",
                backend);
    moe_stager* st = new moe_stager();
    st->backend = backend;
    st->types.resize(n_types);
    for (int i = 0; i < n_types; ++i) {
        Type& t = st->types[i];
        if (n_slots[i] < 1 || slot_bytes[i] == 0 || slot_mem[i] == nullptr) {
            moe::set_error("moe_stage_create: type %d needs >= 1 slot, non-zero slot size and slot memory", i);
            delete st;
            return MOE_ERR_INVALID;
        }
        t.slot_bytes = slot_bytes[i];
        t.n_total = t.n_active = n_slots[i];
        t.mem = static_cast<uint8_t*>(slot_mem[i]);
        t.owner.assign(t.n_total, -1);
        t.freed.assign(t.n_total, nullptr);
        t.freed_pending.assign(t.n_total, 0);
        t.freed_strm.assign(t.n_total, nullptr);
        t.freed_ev.assign(t.n_total, nullptr);
        t.freed_ticket.assign(t.n_total, 0);
        t.freed_valid.assign(t.n_total, 0);
    }
    if (backend == MOE_STAGE_DEVICE) {
        hipError_t e = hipStreamCreateWithFlags(&st->copy_stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            moe::set_error("moe_stage_create: hipStreamCreateWithFlags: %s", hipGetErrorString(e));
            delete st;
            return MOE_ERR_HIP;
        }
        for (Type& t : st->types)
            for (int s = 0; s < t.n_total; ++s) {
                e = hipEventCreateWithFlags(&t.freed[s], hipEventDisableTiming);
                if (e != hipSuccess) {
                    moe::set_error("moe_stage_create: hipEventCreateWithFlags: %s", hipGetErrorString(e));
                    moe_stage_destroy(st);   // releases the stream and the events made so far
                    return MOE_ERR_HIP;
                }
            }
    }
    *out = st;
    return MOE_OK;
}

extern "C" int moe_stage_add_module(moe_stager* st, int32_t type, int32_t n_tensors, const void* const* src,
                                    const size_t* bytes, const size_t* dst_offsets) {
    MOE_REQUIRE(st && src && bytes && dst_offsets, "moe_stage_add_module: NULL argument");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(type >= 0 && type < (int)st->types.size(), "moe_stage_add_module: bad type %d", type);
    MOE_REQUIRE(n_tensors >= 1, "moe_stage_add_module: n_tensors %d < 1", n_tensors);
    Type& t = st->types[type];
    Module m;
    m.type = type;
    for (int i = 0; i < n_tensors; ++i) {
        MOE_REQUIRE(src[i] != nullptr, "moe_stage_add_module: tensor %d has a NULL source", i);
        MOE_REQUIRE(dst_offsets[i] + bytes[i] <= t.slot_bytes,
                    "moe_stage_add_module: tensor %d (%zu bytes at offset %zu) overruns the %zu-byte slot", i, bytes[i],
                    dst_offsets[i], t.slot_bytes);
        m.pieces.push_back(Piece{src[i], bytes[i], dst_offsets[i]});
    }
    if (st->backend == MOE_STAGE_DEVICE) MOE_HIP_CHECK(hipEventCreateWithFlags(&m.ready, hipEventDisableTiming));
    const int id = (int)st->modules.size();
    st->modules.push_back(std::move(m));
    t.order.push_back(id);
    t.fifo.push_back(id);
    return id;
}

extern "C" int moe_stage_set_bounce(moe_stager* st, int32_t n_chunks, size_t chunk_bytes, int32_t n_threads) {
    MOE_REQUIRE(st, "moe_stage_set_bounce: NULL stager");
    MOE_REQUIRE(n_chunks >= 2 && n_chunks <= 256, "moe_stage_set_bounce: n_chunks %d outside [2,256]", n_chunks);
    MOE_REQUIRE(chunk_bytes >= 4096 && chunk_bytes <= ((size_t)1 << 32), "moe_stage_set_bounce: chunk_bytes %zu outside [4096, 4 GiB]",
                chunk_bytes);
    MOE_REQUIRE(n_threads >= 1 && n_threads <= 64, "moe_stage_set_bounce: n_threads %d outside [1,64]", n_threads);
    std::lock_guard<std::mutex> lk(st->mu);
    Bounce& b = st->bounce;
    MOE_REQUIRE(b.n_chunks == 0, "moe_stage_set_bounce: the bounce ring is already configured");
    b.backend = st->backend;
    b.stream = st->copy_stream;
    b.chunk_bytes = chunk_bytes;
    b.n_threads = n_threads;
    if (st->backend == MOE_STAGE_DEVICE) MOE_HIP_CHECK(hipGetDevice(&b.device));
    for (int i = 0; i < n_chunks; ++i) {
        uint8_t* p = nullptr;
        hipEvent_t ev = nullptr;
        if (st->backend == MOE_STAGE_DEVICE) {
            // pinned memory is ALLOCATED here; existing memory is never registered
            hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&p), chunk_bytes, hipHostMallocDefault);
            if (e == hipSuccess) e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
            if (e != hipSuccess) {
                if (p) (void)hipHostFree(p);
                moe::set_error("moe_stage_set_bounce: chunk %d of %zu bytes: %s", i, chunk_bytes, hipGetErrorString(e));
                b.shutdown();
                return MOE_ERR_HIP;
            }
        } else {
            p = static_cast<uint8_t*>(std::malloc(chunk_bytes));
            if (!p) {
                moe::set_error("moe_stage_set_bounce: out of memory for chunk %d", i);
                b.shutdown();
                return MOE_ERR_INVALID;
            }
        }
        b.chunk.push_back(p);
        b.done.push_back(ev);
        b.busy.push_back(0);
    }
    b.n_chunks = n_chunks;
    b.worker = std::thread([&b] { b.loop(); });
    return MOE_OK;
}

extern "C" int moe_stage_add_module_pageable(moe_stager* st, int32_t type, int32_t n_tensors, const void* const* src,
                                             const size_t* bytes, const size_t* dst_offsets) {
    int id = moe_stage_add_module(st, type, n_tensors, src, bytes, dst_offsets);
    if (id < 0) return id;
    std::lock_guard<std::mutex> lk(st->mu);
    st->modules[id].pageable = true;
    return id;
}

extern "C" int moe_stage_pump(moe_stager* st) {
    MOE_REQUIRE(st, "moe_stage_pump: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    return pump_all(st);
}

extern "C" int moe_stage_acquire(moe_stager* st, int32_t id, void* stream, int32_t* slot) {
    MOE_REQUIRE(st && slot, "moe_stage_acquire: NULL argument");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(id >= 0 && id < (int)st->modules.size(), "moe_stage_acquire: unknown module id %d", id);
    Module& m = st->modules[id];
    if (m.slot < 0 && st->types[m.type].policy == MOE_STAGE_ON_DEMAND) {
        int r = fetch_one(st, id);
        if (r < 0) return r;
    }
    while (m.slot < 0) {
        int r = pump_all(st);
        if (r < 0) return r;
        if (r == 0 && m.slot < 0) {
            moe::set_error("moe_stage_acquire: module %d cannot be scheduled: every slot of type %d is held "
                           "(release or clear earlier modules first)", id, m.type);
            return MOE_ERR_STATE;
        }
    }
    if (m.pageable) {   // the worker must have enqueued this module's copies (and recorded `ready`) before anyone waits on it
        int rc = st->bounce.wait_issued(m.job_seq);
        if (rc != MOE_OK) return rc;
    }
    if (st->backend == MOE_STAGE_DEVICE) MOE_HIP_CHECK(hipStreamWaitEvent(moe::as_stream(stream), m.ready, 0));
    if (!m.held) ++st->n_held;
    m.held = true;
    *slot = m.slot;
    return MOE_OK;
}

extern "C" int moe_stage_release(moe_stager* st, int32_t id, void* stream) {
    MOE_REQUIRE(st, "moe_stage_release: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(id >= 0 && id < (int)st->modules.size(), "moe_stage_release: unknown module id %d", id);
    Module& m = st->modules[id];
    if (m.slot < 0) {
        moe::set_error("moe_stage_release: module %d is not resident", id);
        return MOE_ERR_STATE;
    }
    int rc = release_one(st, id, moe::as_stream(stream));
    if (rc != MOE_OK) return rc;
    // The worker refills a freed slot at once -- on the device once the caller has let go of everything it holds: the
    // slots of a wave released one after the other then share one event (flush_released).  While other modules
    // stay held, the refill waits for the next call that copies (acquire, fetch, pump).
    if (st->backend == MOE_STAGE_DEVICE && st->n_held > 0) return MOE_OK;
    int r = pump_all(st);
    return r < 0 ? r : MOE_OK;
}

extern "C" int moe_stage_set_model(moe_stager* st, const char* model_type, int32_t num_hidden_layers,
                                   int32_t num_local_experts) {
    MOE_REQUIRE(st && model_type, "moe_stage_set_model: NULL argument");
    MOE_REQUIRE(num_hidden_layers >= 0 && num_local_experts >= 0, "moe_stage_set_model: negative count");
    std::lock_guard<std::mutex> lk(st->mu);
    // GPU_Weight_Buffer.cpp:279-294: the layers before the first MoE layer's successor wrap to the last layer
    st->wrap_layers = std::strcmp(model_type, "deepseek_v2") == 0 ? 2 : std::strcmp(model_type, "deepseek_v3") == 0 ? 4 : 0;
    st->num_hidden_layers = num_hidden_layers;
    st->num_local_experts = num_local_experts;
    return MOE_OK;
}

extern "C" int moe_stage_tag_module(moe_stager* st, int32_t id, int32_t layer_idx, int32_t expert_idx) {
    MOE_REQUIRE(st, "moe_stage_tag_module: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(id >= 0 && id < (int)st->modules.size(), "moe_stage_tag_module: unknown module id %d", id);
    MOE_REQUIRE(layer_idx >= 0 && expert_idx >= -1, "moe_stage_tag_module: bad tag (layer %d, expert %d)", layer_idx,
                expert_idx);
    st->modules[id].layer = layer_idx;
    st->modules[id].expert = expert_idx;
    return MOE_OK;
}

extern "C" int moe_stage_clear_expert_buffer(moe_stager* st, int32_t layer_idx, int32_t expert_idx, void* stream) {
    MOE_REQUIRE(st, "moe_stage_clear_expert_buffer: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    const int prev = (layer_idx >= 0 && layer_idx < st->wrap_layers) ? st->num_hidden_layers - 1 : layer_idx - 1;
    int n = 0;
    // only resident modules can be released: walk the slots (a few dozen), not the modules (thousands in a model)
    for (Type& t : st->types)
        for (int s = 0; s < t.n_total; ++s) {
            const int id = t.owner[s];
            if (id < 0) continue;
            Module& m = st->modules[id];
            if (m.expert < 0) continue;                                 // not a routed expert
            const bool earlier = m.layer == layer_idx && m.expert < expert_idx;
            const bool previous = m.layer == prev && m.expert < st->num_local_experts;
            if (!earlier && !previous) continue;
            int rc = release_one(st, id, moe::as_stream(stream));
            if (rc != MOE_OK) return rc;
            ++n;
        }
    if (n > 0) {
        int r = pump_all(st);
        if (r < 0) return r;
    }
    return n;
}

extern "C" int moe_stage_set_phase_slots(moe_stager* st, int32_t type, int32_t n_prefill, int32_t n_decoding) {
    MOE_REQUIRE(st, "moe_stage_set_phase_slots: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(type >= 0 && type < (int)st->types.size(), "moe_stage_set_phase_slots: bad type %d", type);
    Type& t = st->types[type];
    MOE_REQUIRE(n_prefill >= 1 && n_prefill <= t.n_total && n_decoding >= n_prefill && n_decoding <= t.n_total,
                "moe_stage_set_phase_slots: need 1 <= prefill %d <= decoding %d <= %d slots", n_prefill, n_decoding,
                t.n_total);
    for (int s = n_prefill; s < t.n_total; ++s)
        MOE_REQUIRE(st->decoding || t.owner[s] < 0, "moe_stage_set_phase_slots: slot %d of type %d is occupied", s, type);
    t.n_prefill = n_prefill;
    t.n_decoding = n_decoding;
    t.n_active = st->decoding ? n_decoding : n_prefill;
    return MOE_OK;
}

extern "C" int moe_stage_set_phase(moe_stager* st, const char* phase) {
    MOE_REQUIRE(st && phase, "moe_stage_set_phase: NULL argument");
    std::lock_guard<std::mutex> lk(st->mu);
    const bool dec = std::strcmp(phase, "decoding") == 0;
    MOE_REQUIRE(dec || std::strcmp(phase, "prefill") == 0, "moe_stage_set_phase: unknown phase '%s'", phase);
    st->decoding = dec ? 1 : 0;
    if (dec)   // resize_buffer: the pools grow to their decoding size; nothing shrinks here
        for (Type& t : st->types)
            if (t.n_decoding > t.n_active) t.n_active = t.n_decoding;
    return MOE_OK;
}

extern "C" int moe_stage_reset_prefill_buffer(moe_stager* st) {
    MOE_REQUIRE(st, "moe_stage_reset_prefill_buffer: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    for (size_t ti = 0; ti < st->types.size(); ++ti) {
        int rc = drop_residency(st, (int)ti, "moe_stage_reset_prefill_buffer");
        if (rc != MOE_OK) return rc;
    }
    for (Type& t : st->types)
        if (t.n_prefill > 0) t.n_active = t.n_prefill;
    return MOE_OK;
}

extern "C" int moe_stage_reset_weight_copy_queue(moe_stager* st) {
    MOE_REQUIRE(st, "moe_stage_reset_weight_copy_queue: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    for (Type& t : st->types) t.fifo.assign(t.order.begin(), t.order.end());
    return MOE_OK;
}

extern "C" int moe_stage_set_policy(moe_stager* st, int32_t type, int32_t policy) {
    MOE_REQUIRE(st, "moe_stage_set_policy: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(type >= 0 && type < (int)st->types.size(), "moe_stage_set_policy: bad type %d", type);
    MOE_REQUIRE(policy == MOE_STAGE_CYCLIC || policy == MOE_STAGE_ON_DEMAND, "moe_stage_set_policy: bad policy %d",
                policy);
    st->types[type].policy = policy;
    return MOE_OK;
}

extern "C" int moe_stage_fetch(moe_stager* st, const int32_t* ids, int32_t n, int32_t* n_enqueued) {
    MOE_REQUIRE(st && (ids || n == 0), "moe_stage_fetch: NULL argument");
    MOE_REQUIRE(n >= 0, "moe_stage_fetch: n %d < 0", n);
    std::lock_guard<std::mutex> lk(st->mu);
    int done = 0;
    for (int i = 0; i < n; ++i) {
        MOE_REQUIRE(ids[i] >= 0 && ids[i] < (int)st->modules.size(), "moe_stage_fetch: unknown module id %d", ids[i]);
        int r = fetch_one(st, ids[i]);
        if (r < 0) {
            if (n_enqueued) *n_enqueued = done;
            return r;
        }
        done += r;
    }
    if (n_enqueued) *n_enqueued = done;
    return MOE_OK;
}

extern "C" int moe_stage_resident(moe_stager* st, int32_t id) {
    MOE_REQUIRE(st, "moe_stage_resident: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(id >= 0 && id < (int)st->modules.size(), "moe_stage_resident: unknown module id %d", id);
    return st->modules[id].slot >= 0 ? 1 : 0;
}

extern "C" int moe_stage_set_active_slots(moe_stager* st, int32_t type, int32_t n_active, int32_t reset) {
    MOE_REQUIRE(st, "moe_stage_set_active_slots: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    MOE_REQUIRE(type >= 0 && type < (int)st->types.size(), "moe_stage_set_active_slots: bad type %d", type);
    Type& t = st->types[type];
    MOE_REQUIRE(n_active >= 1 && n_active <= t.n_total, "moe_stage_set_active_slots: %d outside [1,%d]", n_active,
                t.n_total);
    if (reset) {
        int rc = drop_residency(st, type, "moe_stage_set_active_slots");
        if (rc != MOE_OK) return rc;
        t.fifo.assign(t.order.begin(), t.order.end());
    } else {
        for (int s = n_active; s < t.n_total; ++s)
            if (t.owner[s] >= 0) {
                moe::set_error("moe_stage_set_active_slots: slot %d of type %d is still occupied", s, type);
                return MOE_ERR_STATE;
            }
    }
    t.n_active = n_active;
    return MOE_OK;
}

extern "C" int moe_stage_stats(moe_stager* st, int64_t* n_copies, int64_t* n_bytes) {
    MOE_REQUIRE(st, "moe_stage_stats: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    if (n_copies) *n_copies = st->n_copies;
    if (n_bytes) *n_bytes = st->n_bytes;
    return MOE_OK;
}

extern "C" int moe_stage_sync(moe_stager* st) {
    MOE_REQUIRE(st, "moe_stage_sync: NULL stager");
    std::lock_guard<std::mutex> lk(st->mu);
    if (st->bounce.n_chunks > 0) {
        int rc = st->bounce.wait_issued(st->bounce.enqueued);
        if (rc != MOE_OK) return rc;
    }
    if (st->backend == MOE_STAGE_DEVICE) {
        int rc = flush_released(st);
        if (rc != MOE_OK) return rc;
        MOE_HIP_CHECK(hipStreamSynchronize(st->copy_stream));
    }
    return MOE_OK;
}

extern "C" int moe_stage_destroy(moe_stager* st) {
    if (!st) return MOE_OK;
    st->bounce.shutdown();   // (joins the worker: queued jobs are finished first)
    if (st->backend == MOE_STAGE_DEVICE) {
        (void)hipStreamSynchronize(st->copy_stream);
        for (Module& m : st->modules)
            if (m.ready) (void)hipEventDestroy(m.ready);
        for (Type& t : st->types)
            for (hipEvent_t ev : t.freed)
                if (ev) (void)hipEventDestroy(ev);
        (void)hipStreamDestroy(st->copy_stream);
    }
    delete st;
    return MOE_OK;
}
