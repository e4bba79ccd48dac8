// Device runtime behind the vkJAX jaxpr interpreter on MI355X: contexts, HBM buffers,
// gfx950 code objects and recorded sequences, exported through the C ABI declared in
// include/vkjax_hip.h. Host-only translation unit; kernels live in separate code objects
// that the caller loads with vkj_module_load.
#include "shim_internal.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <thread>
#include <new>
#include <unordered_map>
#include <string>
#include <vector>
#include <algorithm>

namespace vkj {

thread_local std::string g_last_error;

Registry& registry() {
    static Registry r;
    return r;
}

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    g_last_error = std::string(what) + ": " + hipGetErrorString(e);
    return (int)e > 0 ? (int)e : VKJ_EINVAL;
}

}  // namespace vkj

namespace {

using namespace vkj;

// Large uploads: the copy into the pinned staging buffer is done by a few threads, chunk by chunk,
// while the calling thread hands every finished chunk to the DMA engine in order, so that staging
// and transfer overlap instead of running one after the other.
// Measured on this machine for 38.5 MB of arguments (one hipMemcpyAsync from pinned memory: 57 GB/s): 4 MB chunks
// staged by eight threads and sent on one stream 40 GB/s; 1 MB chunks, four threads, chunks alternating between
// two streams 48 GB/s (more staging threads than four only get in each other's way on the host's memory).
constexpr size_t STAGE_CHUNK     = 4u << 20;   // results on their way back
constexpr size_t UPLOAD_CHUNK    = 1u << 20;   // arguments
constexpr size_t STAGE_MIN       = 8u << 20;   // smaller transfers are copied inline
constexpr size_t CHECKPOINT_BYTES = 2u << 20;  // launches that follow the uploads: this much until their first wait behind the first launch, then twice as much each time
constexpr int    STAGE_THREADS   = 8;
constexpr int    UPLOAD_THREADS  = 4;

template <class Issue>
int staged_upload(char* staging, const char* host, size_t nbytes, Issue&& issue) {
    constexpr size_t STAGE_CHUNK = UPLOAD_CHUNK;
    constexpr int    STAGE_THREADS = UPLOAD_THREADS;
    const size_t nchunks = (nbytes + STAGE_CHUNK - 1) / STAGE_CHUNK;
    std::vector<std::atomic<int>> done(nchunks);
    for (auto& d : done) d.store(0, std::memory_order_relaxed);
    std::atomic<size_t> next{0};
    auto worker = [&]() {
        for (;;) {
            const size_t k = next.fetch_add(1, std::memory_order_relaxed);
            if (k >= nchunks) return;
            const size_t off = k * STAGE_CHUNK, len = std::min(STAGE_CHUNK, nbytes - off);
            memcpy(staging + off, host + off, len);
            done[k].store(1, std::memory_order_release);
        }
    };
    std::vector<std::thread> threads;
    const int nthreads = (int)std::min<size_t>(STAGE_THREADS, nchunks);
    try {
        for (int t = 0; t < nthreads; t++) threads.emplace_back(worker);
    } catch (...) {
        // no (more) threads to be had: the calling thread copies whatever is left
    }
    if ((int)threads.size() < nthreads) worker();
    int status = 0;
    for (size_t k = 0; k < nchunks; k++) {
        while (!done[k].load(std::memory_order_acquire)) std::this_thread::yield();
        const size_t off = k * STAGE_CHUNK, len = std::min(STAGE_CHUNK, nbytes - off);
        if (status == 0) status = issue(off, len);
    }
    for (auto& t : threads) t.join();
    return status;
}

// The same for all arguments of an evaluation together (a network's weights: hundreds of arrays of a few MB each,
// which one thread would stage one after the other at the speed of a single core's memcpy).
struct UploadPiece { char* staging; const char* host; char* device; size_t nbytes; };

template <class Issue>
int staged_upload_pieces(const std::vector<UploadPiece>& pieces, Issue&& issue) {
    constexpr size_t STAGE_CHUNK = UPLOAD_CHUNK;
    constexpr int    STAGE_THREADS = UPLOAD_THREADS;
    struct Chunk { size_t piece, off, len; };
    std::vector<Chunk> chunks;
    for (size_t p = 0; p < pieces.size(); p++)
        for (size_t off = 0; off < pieces[p].nbytes; off += STAGE_CHUNK)
            chunks.push_back({p, off, std::min(STAGE_CHUNK, pieces[p].nbytes - off)});
    const size_t nchunks = chunks.size();
    std::vector<std::atomic<int>> done(nchunks);
    for (auto& d : done) d.store(0, std::memory_order_relaxed);
    std::atomic<size_t> next{0};
    auto worker = [&]() {
        for (;;) {
            const size_t k = next.fetch_add(1, std::memory_order_relaxed);
            if (k >= nchunks) return;
            const Chunk& ch = chunks[k];
            memcpy(pieces[ch.piece].staging + ch.off, pieces[ch.piece].host + ch.off, ch.len);
            done[k].store(1, std::memory_order_release);
        }
    };
    std::vector<std::thread> threads;
    const int nthreads = (int)std::min<size_t>(STAGE_THREADS, nchunks);
    try {
        for (int t = 0; t < nthreads; t++) threads.emplace_back(worker);
    } catch (...) {
        // no (more) threads to be had: the calling thread copies whatever is left
    }
    if ((int)threads.size() < nthreads) worker();
    int status = 0;
    for (size_t k = 0; k < nchunks; k++) {
        while (!done[k].load(std::memory_order_acquire)) std::this_thread::yield();
        const Chunk& ch = chunks[k];
        if (status == 0) status = issue(k, ch.piece, ch.off, ch.len);
    }
    for (auto& t : threads) t.join();
    return status;
}

// Large downloads, the other way round: the transfer is issued chunk by chunk with an event behind every
// chunk; the calling thread waits for the events in order and a few threads copy each chunk out of the
// pinned buffer as soon as it has landed, while the chunks after it are still on their way.
template <class Wait>
int staged_copy_out(char* dst, const char* staging, size_t nbytes, Wait&& wait_for_chunk) {
    const size_t nchunks = (nbytes + STAGE_CHUNK - 1) / STAGE_CHUNK;
    std::atomic<size_t> landed{0}, next{0};
    auto worker = [&]() {
        for (;;) {
            const size_t k = next.fetch_add(1, std::memory_order_relaxed);
            if (k >= nchunks) return;
            while (landed.load(std::memory_order_acquire) <= k) std::this_thread::yield();
            const size_t off = k * STAGE_CHUNK;
            memcpy(dst + off, staging + off, std::min(STAGE_CHUNK, nbytes - off));
        }
    };
    std::vector<std::thread> threads;
    try {
        for (int t = 0; t < (int)std::min<size_t>(STAGE_THREADS, nchunks); t++) threads.emplace_back(worker);
    } catch (...) {
    }
    int status = 0;
    for (size_t k = 0; k < nchunks; k++) {
        if (status == 0) status = wait_for_chunk(k);
        landed.store(k + 1, std::memory_order_release);      // after a failure too: the helpers must come to an end
    }
    if (threads.empty()) worker();
    for (auto& t : threads) t.join();
    return status;
}

int use(Ctx* c) {
    HIP_TRY(hipSetDevice(c->device));
    return 0;
}

void destroy_ctx_objects(Ctx* c) {
    if (c->ev_begin)    hipEventDestroy(c->ev_begin);
    if (c->ev_end)      hipEventDestroy(c->ev_end);
    if (c->ev_landed)   hipEventDestroy(c->ev_landed);
    if (c->ev_uploaded) hipEventDestroy(c->ev_uploaded);
    if (c->ev_copied)   hipEventDestroy(c->ev_copied);
    if (c->stream)      hipStreamDestroy(c->stream);
    if (c->copy_stream) hipStreamDestroy(c->copy_stream);
    for (auto& e : c->ev_checkpoint) { if (e) hipEventDestroy(e); e = nullptr; }
    if (c->side_stream) hipStreamDestroy(c->side_stream);
    c->ev_begin = c->ev_end = c->ev_landed = c->ev_uploaded = c->ev_copied = nullptr;
    c->stream = c->copy_stream = c->side_stream = nullptr;
}

// A sequence lets go of a buffer it recorded; the memory of a buffer that vkj_buf_free has
// already been called on is released with the last such reference.
// The device memory of a buffer goes: its own allocation, or its share of a slab (the slab with its last array).
hipError_t free_buf_memory(Buf* b) {
    if (!b->slab) return hipFree(b->dptr);
    Slab* slab = b->slab;
    b->slab = nullptr;
    if (--slab->live > 0) return hipSuccess;
    auto& slabs = b->ctx->slabs;
    slabs.erase(std::remove(slabs.begin(), slabs.end(), slab), slabs.end());
    hipError_t e = hipFree(slab->base);
    delete slab;
    return e;
}

void unref_buf(Buf* b) {
    if (--b->seq_refs == 0 && b->released) {
        free_buf_memory(b);
        delete b;
    }
}

int issue_launch(Ctx* c, Launch& l, hipStream_t stream = nullptr) {
    size_t size = l.kernarg.size();
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, l.kernarg.data(),
                     HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    hipError_t e = hipModuleLaunchKernel(l.fn->fn, l.grid[0], l.grid[1], l.grid[2],
                                         l.block[0], l.block[1], l.block[2], l.lds, stream ? stream : c->stream, nullptr, extra);
    if (e != hipSuccess) {
        g_last_error = "launch of " + l.fn->name + ": " + hipGetErrorString(e);
        return (int)e;
    }
    return 0;
}

void drop_graph(Seq* s) {
    if (s->graph_exec) { hipGraphExecDestroy(s->graph_exec); s->graph_exec = nullptr; }
    s->graph_failed = false;
}

// All launches of a sequence, once: as its captured graph when that is asked for, else one by one. `first`: the
// launches before it have been issued already (the first launch, in parts, beside the uploads).
int issue_all(Ctx* c, Seq* s, size_t first = 0) {
    if (first) {
        for (size_t i = first; i < s->launches.size(); i++)
            if (int r = issue_launch(c, s->launches[i])) return r;
        return 0;
    }
    if (s->want_graph && !s->profiling && !s->graph_failed && s->launches.size() > 1) {
        if (!s->graph_exec) {
            hipGraph_t graph = nullptr;
            hipError_t e = hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal);
            if (e == hipSuccess) {
                int r = 0;
                for (auto& l : s->launches) if ((r = issue_launch(c, l))) break;
                hipError_t e2 = hipStreamEndCapture(c->stream, &graph);
                if (r == 0 && e2 == hipSuccess && graph) e = hipGraphInstantiate(&s->graph_exec, graph, nullptr, nullptr, 0);
                else e = e2 == hipSuccess ? hipErrorUnknown : e2;
                if (graph) hipGraphDestroy(graph);
            }
            if (e != hipSuccess || !s->graph_exec) {
                (void)hipGetLastError();
                s->graph_exec = nullptr;
                s->graph_failed = true;
            }
        }
        if (s->graph_exec) {
            HIP_TRY(hipGraphLaunch(s->graph_exec, c->stream));
            return 0;
        }
    }
    if (!s->uses_side) {
        for (auto& l : s->launches)
            if (int r = issue_launch(c, l)) return r;
        return 0;
    }
    // Two lanes: launches keep their recorded order on each lane's stream; where a launch was told to wait for the
    // other lane, an event recorded there (behind everything issued on it so far) is waited for on its own lane
    // first. Lane 1 starts behind what the stream holds already (the uploads) and is joined at the end, so that
    // whatever follows on the stream - downloads, the final wait - follows both. (A captured graph and a sequence
    // with time stamps issue every launch on the stream, in recorded order, which satisfies the same dependencies.)
    HIP_TRY(hipEventRecord(s->ev_fork, c->stream));
    HIP_TRY(hipStreamWaitEvent(c->side_stream, s->ev_fork, 0));
    for (auto& l : s->launches) {
        hipStream_t mine = l.lane ? c->side_stream : c->stream, other = l.lane ? c->stream : c->side_stream;
        if (l.wait_event) {
            HIP_TRY(hipEventRecord(l.wait_event, other));
            HIP_TRY(hipStreamWaitEvent(mine, l.wait_event, 0));
        }
        if (int r = issue_launch(c, l, mine)) return r;
    }
    HIP_TRY(hipEventRecord(s->ev_join, c->side_stream));
    HIP_TRY(hipStreamWaitEvent(c->stream, s->ev_join, 0));
    return 0;
}

}  // namespace

int vkj::seq_eval(Seq* s, void* const* host_ptrs, int nslots, uint32_t flags, void* const* next_host_ptrs,
                  const LandingRegion* region) {
    Ctx* c = s->ctx;
    if (int r = use(c)) return r;
    const bool up = !(flags & VKJ_EVAL_SKIP_UPLOADS), down = !(flags & VKJ_EVAL_SKIP_DOWNLOADS);
    auto slot_ok = [&](const Transfer& t) { return t.nbytes == 0 || (host_ptrs && t.slot < nslots && host_ptrs[t.slot]); };
    const bool null_resident = flags & VKJ_EVAL_NULL_IS_RESIDENT;
    if (up)   for (auto& t : s->uploads)   if (!slot_ok(t) && !(null_resident && host_ptrs && t.slot < nslots))
        return fail(VKJ_EINVAL, "vkj_seq_eval: no host pointer for upload slot %d", t.slot);
    if (down) for (auto& t : s->downloads) if (!slot_ok(t)) return fail(VKJ_EINVAL, "vkj_seq_eval: no host pointer for download slot %d", t.slot);

    size_t nstamps = 0, first_launch = 0;        // first_launch: 1 when the first launch has been issued in parts beside the uploads
    bool launches_issued = false;                // all of them, beside the uploads
    if (s->profiling) {
        nstamps = 3 + s->launches.size();       // begin, after uploads, after each launch, after downloads
        while (s->stamps.size() < nstamps) {
            hipEvent_t e;
            HIP_TRY(hipEventCreate(&e));
            s->stamps.push_back(e);
        }
        s->stamps_valid = 0;
        HIP_TRY(hipEventRecord(s->stamps[0], c->stream));
    }
    if (up) {
        size_t total = 0;
        for (auto& t : s->uploads) if (t.nbytes && host_ptrs[t.slot]) total += t.nbytes;
        if (total >= STAGE_MIN) {
            // all arguments as one stream of chunks: a few threads stage them, this one hands each chunk to the
            // DMA engine as soon as it is staged
            std::vector<UploadPiece> pieces;
            std::vector<int> piece_slot;
            for (auto& t : s->uploads)
                if (t.nbytes && host_ptrs[t.slot]) {
                    pieces.push_back({(char*)t.staging, (const char*)host_ptrs[t.slot], (char*)t.buf->dptr + t.offset, t.nbytes});
                    piece_slot.push_back(t.slot);
                }
            const size_t nl = s->launches.size();
            // Launches that follow the uploads: a program that brings all its weights with every call need not wait for
            // the last of them before its first layer starts. The arguments travel in the order in which the launches
            // first read them (the arrays of one launch smallest first), over two streams that carry nothing else, and
            // at a few checkpoints along the way the launch stream is told to wait for what has been handed over so
            // far and is given the launches that read nothing beyond it. (Not with time stamps, a captured graph, a
            // second lane or a fixed landing region, whose bookkeeping assumes the uploads are over before the launches.)
            const bool follow = nl > 0 && !s->profiling && !s->want_graph && !s->uses_side && !region;
            std::vector<long> need(nl, -1);              // the last piece (in sending order) a launch or any launch before it reads
            std::vector<size_t> checkpoints;             // pieces behind which launches are issued, ascending; the last piece is one
            if (follow) {
                std::vector<size_t> first_use(pieces.size(), nl), order(pieces.size());
                std::unordered_multimap<const void*, size_t> piece_of;          // device allocation -> pieces that land in it
                {
                    size_t p = 0;
                    for (auto& t : s->uploads) if (t.nbytes && host_ptrs[t.slot]) piece_of.emplace(t.buf, p++);
                }
                for (size_t i = 0; i < nl; i++)
                    for (Buf* b : s->launches[i].bufs) {
                        auto range = piece_of.equal_range(b);
                        for (auto it = range.first; it != range.second; ++it) first_use[it->second] = std::min(first_use[it->second], i);
                    }
                // (small arrays first, in the order they were recorded in: together they are a fraction of a megabyte, and
                // neighbours in memory stay neighbours on the way, which lets one transfer carry a run of them)
                for (size_t p = 0; p < order.size(); p++) {
                    order[p] = p;
                    if (pieces[p].nbytes <= PACKED_MAX_BYTES) first_use[p] = 0;
                }
                std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) {
                    const bool small_a = pieces[a].nbytes <= PACKED_MAX_BYTES, small_b = pieces[b].nbytes <= PACKED_MAX_BYTES;
                    if (small_a != small_b) return small_a;
                    if (small_a) return false;
                    return first_use[a] != first_use[b] ? first_use[a] < first_use[b] : pieces[a].nbytes < pieces[b].nbytes;
                });
                std::vector<UploadPiece> sorted_pieces;
                std::vector<int> sorted_slot;
                std::vector<size_t> sorted_use;
                for (size_t p : order) { sorted_pieces.push_back(pieces[p]); sorted_slot.push_back(piece_slot[p]); sorted_use.push_back(first_use[p]); }
                pieces.swap(sorted_pieces);
                piece_slot.swap(sorted_slot);
                // (sorted by first use: the pieces a launch needs end where the pieces first read by a later launch begin)
                size_t p = 0;
                long reached = -1;
                for (size_t i = 0; i < nl; i++) {
                    while (p < pieces.size() && sorted_use[p] <= i) reached = (long)p++;
                    need[i] = reached;
                }
                // the first checkpoint lets the first launch go; behind it a handful, the distance doubling from
                // CHECKPOINT_BYTES on (the first layers of a network read little and should not wait for much)
                if (need[0] >= 0 && (size_t)need[0] + 1 < pieces.size()) checkpoints.push_back((size_t)need[0]);
                size_t since = 0, step = CHECKPOINT_BYTES;
                for (size_t q = (size_t)(need[0] + 1); q + 1 < pieces.size(); q++) {
                    since += pieces[q].nbytes;
                    if (since >= step && (int)checkpoints.size() < Ctx::MAX_CHECKPOINTS - 1) { checkpoints.push_back(q); since = 0; step *= 2; }
                }
                checkpoints.push_back(pieces.size() - 1);
            }
            // Without that the chunks alternate between the launch stream and the copy stream (two copy engines work on
            // them) and the launches wait for both. All streams are idle here: every evaluation ends with everything
            // it queued on them complete.
            hipStream_t copy_even = follow ? c->side_stream : c->stream, copy_odd = c->copy_stream;
            // (the parts of the first launch: on the side stream beside chunks on the launch stream, or - the side stream
            // carrying chunks - on the launch stream itself, which has nothing else to do until the first checkpoint)
            hipStream_t parts_stream = follow ? c->stream : c->side_stream;
            // The first launch in parts: a part goes to the side stream as soon as the chunks it reads have been
            // handed to the copy engines (both streams are in order: an event behind a chunk covers every chunk
            // before it), so the device computes while the rest of the argument is still on its way. Only with that
            // argument as the last thing the first launch reads to be sent: whatever else it reads has then been sent.
            size_t early_piece = pieces.size(), next_part = 0;
            if (!s->early.empty() && !s->profiling && !s->want_graph && !s->uses_side) {
                for (size_t p = 0; p < pieces.size(); p++)
                    if (piece_slot[p] == s->early_slot && pieces[p].nbytes >= s->early.back().bytes_needed) early_piece = p;
                const size_t must_be = follow ? (size_t)(need[0] < 0 ? pieces.size() : need[0]) : pieces.size() - 1;
                if (early_piece != must_be) early_piece = pieces.size();
            }
            hipError_t err = hipSuccess;
            int launch_status = 0;
            size_t next_launch = 0, next_checkpoint = 0;
            // launches that read nothing of this evaluation's uploads, and nothing behind such launches, need not wait at all
            while (follow && next_launch < nl && need[next_launch] < 0) {
                if ((launch_status = issue_launch(c, s->launches[next_launch++]))) return launch_status;
            }
            // Small arrays that lie next to each other in HBM and in their staging memory alike (vkj_buf_alloc_packed) are
            // sent as one transfer: the run is extended while the next array starts within the alignment step behind it,
            // by the same distance on both sides. Hundreds of transfers of a few KB each would cost more host time than
            // the bytes take to travel.
            struct { uintptr_t device = 0, staging = 0; size_t len = 0; hipStream_t stream = nullptr; } run;
            auto flush_run = [&]() {
                if (run.len) err = hipMemcpyAsync((void*)run.device, (const void*)run.staging, run.len, hipMemcpyHostToDevice, run.stream);
                run.len = 0;
                return err == hipSuccess;
            };
            const int r = staged_upload_pieces(pieces, [&](size_t k, size_t piece, size_t off, size_t len) {
                const uintptr_t device = (uintptr_t)(pieces[piece].device + off), staging = (uintptr_t)(pieces[piece].staging + off);
                hipStream_t to = (k & 1) ? copy_odd : copy_even;
                if (pieces[piece].nbytes <= PACKED_MAX_BYTES) {
                    const size_t step = device - run.device;
                    if (run.len && device > run.device && step == staging - run.staging && step >= run.len && step < run.len + PACKED_ALIGN
                            && step + len <= UPLOAD_CHUNK) {
                        run.len = step + len;
                    } else {
                        if (!flush_run()) return 1;
                        run.device = device; run.staging = staging; run.len = len; run.stream = to;
                    }
                } else {
                    if (!flush_run()) return 1;
                    err = hipMemcpyAsync((void*)device, (const void*)staging, len, hipMemcpyHostToDevice, to);
                    if (err != hipSuccess) return 1;
                }
                const bool part_due = piece == early_piece && next_part < s->early.size() && s->early[next_part].bytes_needed <= off + len;
                const bool checkpoint_due = follow && next_checkpoint < checkpoints.size() && piece == checkpoints[next_checkpoint]
                                            && off + len == pieces[piece].nbytes;
                if ((part_due || checkpoint_due) && !flush_run()) return 1;
                while (piece == early_piece && next_part < s->early.size() && s->early[next_part].bytes_needed <= off + len) {
                    EarlyPart& part = s->early[next_part++];
                    if ((err = hipEventRecord(part.ev_a, copy_even)) != hipSuccess) return 1;
                    if ((err = hipEventRecord(part.ev_b, copy_odd)) != hipSuccess) return 1;
                    if ((err = hipStreamWaitEvent(parts_stream, part.ev_a, 0)) != hipSuccess) return 1;
                    if ((err = hipStreamWaitEvent(parts_stream, part.ev_b, 0)) != hipSuccess) return 1;
                    if ((launch_status = issue_launch(c, part.launch, parts_stream))) return 1;
                }
                if (follow && next_checkpoint < checkpoints.size() && piece == checkpoints[next_checkpoint] && off + len == pieces[piece].nbytes) {
                    hipEvent_t ev_even = c->ev_checkpoint[2 * next_checkpoint], ev_odd = c->ev_checkpoint[2 * next_checkpoint + 1];
                    next_checkpoint++;
                    if ((err = hipEventRecord(ev_even, copy_even)) != hipSuccess) return 1;
                    if ((err = hipEventRecord(ev_odd, copy_odd)) != hipSuccess) return 1;
                    if ((err = hipStreamWaitEvent(c->stream, ev_even, 0)) != hipSuccess) return 1;
                    if ((err = hipStreamWaitEvent(c->stream, ev_odd, 0)) != hipSuccess) return 1;
                    // (every part of the first launch has been issued, on this stream: the last one needs no more than the whole argument)
                    if (piece == early_piece && next_launch == 0) next_launch = 1;
                    while (next_launch < nl && need[next_launch] <= (long)piece)
                        if ((launch_status = issue_launch(c, s->launches[next_launch++]))) return 1;
                }
                return 0;
            });
            if (launch_status) return launch_status;
            if (r || !flush_run()) return hip_fail(err, "hipMemcpyAsync (staged upload)");
            if (follow) {
                first_launch = next_launch;          // all of them: the last checkpoint is the last piece
                if (first_launch != nl) return fail(VKJ_ESTATE, "vkj_seq_eval: %zu of %zu launches issued beside the uploads", first_launch, nl);
                launches_issued = true;
            } else {
                HIP_TRY(hipEventRecord(c->ev_copied, c->copy_stream));
                HIP_TRY(hipStreamWaitEvent(c->stream, c->ev_copied, 0));
                if (early_piece < pieces.size()) {
                    // (every part has been issued: the last one needs no more than the whole argument)
                    HIP_TRY(hipEventRecord(s->ev_early_done, c->side_stream));
                    HIP_TRY(hipStreamWaitEvent(c->stream, s->ev_early_done, 0));
                    first_launch = 1;
                }
            }
        } else {
            for (auto& t : s->uploads) {
                if (!t.nbytes || !host_ptrs[t.slot]) continue;
                memcpy(t.staging, host_ptrs[t.slot], t.nbytes);
                HIP_TRY(hipMemcpyAsync((char*)t.buf->dptr + t.offset, t.staging, t.nbytes, hipMemcpyHostToDevice, c->stream));
            }
        }
    }
    if (s->profiling) HIP_TRY(hipEventRecord(s->stamps[1], c->stream));
    // With a fixed landing region nothing is allocated: the following arguments are staged in the
    // upload's own pinned buffer, which must have been emptied by this evaluation's upload first.
    bool staging_in_use = false;
    if (region && next_host_ptrs && up)
        for (auto& t : s->uploads)
            if (t.nbytes && t.slot < nslots && next_host_ptrs[t.slot] && host_ptrs && host_ptrs[t.slot]) staging_in_use = true;
    if (staging_in_use) HIP_TRY(hipEventRecord(c->ev_uploaded, c->stream));
    if (s->profiling) {
        for (size_t i = 0; i < s->launches.size(); i++) {
            if (int r = issue_launch(c, s->launches[i])) return r;
            HIP_TRY(hipEventRecord(s->stamps[2 + i], c->stream));
        }
    } else if (!launches_issued) {
        if (int r = issue_all(c, s, first_launch)) return r;
    }
    bool landed = false;
    if (next_host_ptrs) {
        // While the device works through the launches: stage the following evaluation's arguments and
        // send them, on the second stream, to landing buffers; once the launches are through, move
        // them on into the argument buffers with device-to-device copies.
        bool any = false;
        size_t region_used = 0;
        if (staging_in_use) HIP_TRY(hipEventSynchronize(c->ev_uploaded));
        for (auto& t : s->uploads) {
            if (!t.nbytes || t.slot >= nslots || !next_host_ptrs[t.slot]) continue;
            char *staging, *landing;
            if (region) {
                staging = (char*)t.staging;
                landing = region->base + region_used;       // the caller has checked that everything fits
                region_used += (t.nbytes + 255) & ~(size_t)255;
            } else {
                if (!t.landing) {
                    void *device = nullptr, *pinned = nullptr;
                    HIP_TRY(hipMalloc(&device, t.nbytes));
                    hipError_t e = hipHostMalloc(&pinned, t.nbytes, hipHostMallocDefault);
                    if (e != hipSuccess) { hipFree(device); return hip_fail(e, "hipHostMalloc (staging of the next arguments)"); }
                    t.landing = device;
                    t.next_staging = pinned;
                }
                staging = (char*)t.next_staging;
                landing = (char*)t.landing;
            }
            hipError_t err = hipSuccess;
            auto send = [&](size_t off, size_t len) {
                err = hipMemcpyAsync(landing + off, staging + off, len, hipMemcpyHostToDevice, c->copy_stream);
                return err == hipSuccess ? 0 : 1;
            };
            if (t.nbytes >= STAGE_MIN) {
                if (staged_upload(staging, (const char*)next_host_ptrs[t.slot], t.nbytes, send))
                    return hip_fail(err, "hipMemcpyAsync (staged upload of the next arguments)");
            } else {
                memcpy(staging, next_host_ptrs[t.slot], t.nbytes);
                if (send(0, t.nbytes)) return hip_fail(err, "hipMemcpyAsync (upload of the next arguments)");
            }
            any = true;
        }
        landed = any;
    }
    // The downloads are queued after the copies above on purpose: a copy engine works through its
    // queue in order, and a download queued first waits there for the launches, with every upload
    // behind it, even one from the other stream, waiting as well.
    size_t nchunk_events = 0;
    if (down) for (auto& t : s->downloads) {
        if (!t.nbytes) continue;
        if (t.nbytes < STAGE_MIN) {
            HIP_TRY(hipMemcpyAsync(t.staging, (char*)t.buf->dptr + t.offset, t.nbytes, hipMemcpyDeviceToHost, c->stream));
            continue;
        }
        for (size_t off = 0; off < t.nbytes; off += STAGE_CHUNK, nchunk_events++) {
            HIP_TRY(hipMemcpyAsync((char*)t.staging + off, (char*)t.buf->dptr + t.offset + off, std::min(STAGE_CHUNK, t.nbytes - off),
                                   hipMemcpyDeviceToHost, c->stream));
            HIP_TRY(hipEventRecord(s->chunk_events[nchunk_events], c->stream));
        }
    }
    if (s->profiling) HIP_TRY(hipEventRecord(s->stamps[nstamps - 1], c->stream));
    if (landed) {
        HIP_TRY(hipEventRecord(c->ev_landed, c->copy_stream));
        HIP_TRY(hipStreamWaitEvent(c->stream, c->ev_landed, 0));
        size_t region_used = 0;
        for (auto& t : s->uploads) {
            if (!t.nbytes || t.slot >= nslots || !next_host_ptrs[t.slot]) continue;
            if (region) {
                if (int r = region->move((char*)t.buf->dptr + t.offset, region->base + region_used, t.nbytes, c->stream)) return r;
                region_used += (t.nbytes + 255) & ~(size_t)255;
            } else {
                HIP_TRY(hipMemcpyAsync((char*)t.buf->dptr + t.offset, t.landing, t.nbytes, hipMemcpyDeviceToDevice, c->stream));
            }
        }
    }
    // large results leave the pinned buffers chunk by chunk as they land; then everything else is waited for
    if (down) {
        size_t first_event = 0;
        for (auto& t : s->downloads) {
            if (t.nbytes < STAGE_MIN) continue;
            hipError_t err = hipSuccess;
            const int r = staged_copy_out((char*)host_ptrs[t.slot], (const char*)t.staging, t.nbytes, [&](size_t k) {
                err = hipEventSynchronize(s->chunk_events[first_event + k]);
                return err == hipSuccess ? 0 : 1;
            });
            if (r) return hip_fail(err, "hipEventSynchronize (staged download)");
            first_event += (t.nbytes + STAGE_CHUNK - 1) / STAGE_CHUNK;
        }
    }
    HIP_TRY(hipStreamSynchronize(c->stream));
    if (down) for (auto& t : s->downloads)
        if (t.nbytes && t.nbytes < STAGE_MIN) memcpy(host_ptrs[t.slot], t.staging, t.nbytes);
    if (s->profiling) s->stamps_valid = (int)nstamps;
    return 0;
}

int vkj::seq_eval_static(Seq* s, void* const* host_ptrs, int nslots, uint32_t flags, void* const* next_host_ptrs,
                         int (*move)(void* dst, const void* src, size_t nbytes, hipStream_t stream)) {
    if (s->profiling)
        return fail(VKJ_ESTATE, "vkj_seq_eval_next_static: a sequence with timestamps creates events when evaluated; use vkj_seq_eval_next");
    // the same condition under which issue_all would build the graph (a single launch is never captured)
    if (s->want_graph && !s->graph_failed && s->launches.size() > 1 && !s->graph_exec)
        return fail(VKJ_ESTATE, "vkj_seq_eval_next_static: the sequence's graph has not been built yet (that allocates); "
                                "evaluate it once with vkj_seq_eval first");
    size_t needed = 0;
    if (next_host_ptrs)
        for (auto& t : s->uploads)
            if (t.nbytes && t.slot < nslots && next_host_ptrs[t.slot]) needed += (t.nbytes + 255) & ~(size_t)255;
    if (needed > (size_t)VKJ_STATIC_LANDING_BYTES)
        return fail(VKJ_EINVAL, "vkj_seq_eval_next_static: the following evaluation's arguments take %zu bytes, the static landing "
                                "array holds %zu; use vkj_seq_eval_next", needed, (size_t)VKJ_STATIC_LANDING_BYTES);
    // one array per GPU, shared by every context and thread of the process: claimed for the whole call
    static std::atomic<bool> busy[64];
    std::atomic<bool>& mine = busy[(unsigned)s->ctx->device % 64u];
    if (mine.exchange(true, std::memory_order_acquire))
        return fail(VKJ_ESTATE, "vkj_seq_eval_next_static: static landing array busy (another call on device %d is using it)", s->ctx->device);
    const LandingRegion region{(char*)s->ctx->static_landing, (size_t)VKJ_STATIC_LANDING_BYTES, move};
    const int r = seq_eval(s, host_ptrs, nslots, flags, next_host_ptrs, &region);
    mine.store(false, std::memory_order_release);
    return r;
}

extern "C" {

const char* vkj_last_error(void) { return g_last_error.c_str(); }

int vkj_device_count(int* count) {
    if (!count) return fail(VKJ_EINVAL, "vkj_device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) { *count = 0; return hip_fail(e, "hipGetDeviceCount"); }
    *count = n;
    return 0;
}

int vkj_ctx_create(int device, vkj_handle* out) {
    if (!out) return fail(VKJ_EINVAL, "vkj_ctx_create: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) return fail(VKJ_ENODEV, "vkj_ctx_create: no HIP device available (%s)",
                                               e != hipSuccess ? hipGetErrorString(e) : "count is 0");
    if (device < 0 || device >= n) return fail(VKJ_EINVAL, "vkj_ctx_create: device %d out of range [0,%d)", device, n);
    Ctx* c = new (std::nothrow) Ctx();
    if (!c) return fail(VKJ_ENOMEM, "vkj_ctx_create: out of host memory");
    c->device = device;
    // everything an evaluation needs besides its own buffers is made here, so that none of the
    // evaluation entry points has to create a stream or an event
    int r = [&]() -> int {
        HIP_TRY(hipSetDevice(device));
        HIP_TRY(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
        HIP_TRY(hipStreamCreateWithFlags(&c->copy_stream, hipStreamNonBlocking));
        HIP_TRY(hipStreamCreateWithFlags(&c->side_stream, hipStreamNonBlocking));
        for (auto& e : c->ev_checkpoint) HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        HIP_TRY(hipEventCreate(&c->ev_begin));
        HIP_TRY(hipEventCreate(&c->ev_end));
        HIP_TRY(hipEventCreateWithFlags(&c->ev_landed, hipEventDisableTiming));
        HIP_TRY(hipEventCreateWithFlags(&c->ev_uploaded, hipEventDisableTiming));
        HIP_TRY(hipEventCreateWithFlags(&c->ev_copied, hipEventDisableTiming));
        return static_landing_init(c);
    }();
    if (r) {
        destroy_ctx_objects(c);
        delete c;
        return r;
    }
    *out = to_handle(c);
    return 0;
}

int vkj_ctx_destroy(vkj_handle h) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c) return fail(VKJ_EINVAL, "vkj_ctx_destroy: bad context handle");
    if (int r = use(c)) return r;
    hipStreamSynchronize(c->stream);
    hipStreamSynchronize(c->copy_stream);
    hipStreamSynchronize(c->side_stream);
    destroy_ctx_objects(c);
    retire(c);
    delete c;
    return 0;
}

int vkj_device_props(vkj_handle h, vkj_props* out) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c || !out) return fail(VKJ_EINVAL, "vkj_device_props: bad argument");
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, c->device));
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", p.name);
    snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
    out->compute_units         = p.multiProcessorCount;
    out->wavefront_size        = p.warpSize;
    out->max_threads_per_block = p.maxThreadsPerBlock;
    out->max_block_dim_x       = p.maxThreadsDim[0];
    out->lds_bytes_per_block   = (int32_t)p.sharedMemPerBlock;
    out->clock_khz             = p.clockRate;
    out->memory_clock_khz      = p.memoryClockRate;
    out->memory_bus_bits       = p.memoryBusWidth;
    out->hbm_bytes             = p.totalGlobalMem;
    return 0;
}

int vkj_sync(vkj_handle h) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c) return fail(VKJ_EINVAL, "vkj_sync: bad context handle");
    if (int r = use(c)) return r;
    HIP_TRY(hipStreamSynchronize(c->stream));
    return 0;
}

int vkj_module_load(vkj_handle h, const void* image, size_t nbytes, vkj_handle* out) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c || !image || !nbytes || !out) return fail(VKJ_EINVAL, "vkj_module_load: bad argument");
    if (int r = use(c)) return r;
    Mod* m = new (std::nothrow) Mod();
    if (!m) return fail(VKJ_ENOMEM, "vkj_module_load: out of host memory");
    m->ctx = c;
    hipError_t e = hipModuleLoadData(&m->module, image);
    if (e != hipSuccess) { delete m; return hip_fail(e, "hipModuleLoadData (is the code object built for this GPU's architecture?)"); }
    *out = to_handle(m);
    return 0;
}

int vkj_module_unload(vkj_handle h, vkj_handle mh) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Mod* m = from_handle<Mod>(mh, MAGIC_MOD);
    if (!c || !m || m->ctx != c) return fail(VKJ_EINVAL, "vkj_module_unload: bad handle");
    if (m->seq_refs > 0)
        return fail(VKJ_ESTATE, "vkj_module_unload: %d recorded launch(es) of live sequences use this module; destroy those sequences first",
                    m->seq_refs);
    if (int r = use(c)) return r;
    HIP_TRY(hipStreamSynchronize(c->stream));
    HIP_TRY(hipModuleUnload(m->module));
    // the module's function handles go with it: a later use of one is rejected as a bad handle
    for (Fn* f : m->functions) { retire(f); delete f; }
    retire(m);
    delete m;
    return 0;
}

int vkj_module_get_function(vkj_handle h, vkj_handle mh, const char* name, vkj_handle* out) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Mod* m = from_handle<Mod>(mh, MAGIC_MOD);
    if (!c || !m || m->ctx != c || !name || !out) return fail(VKJ_EINVAL, "vkj_module_get_function: bad argument");
    if (int r = use(c)) return r;
    Fn* f = new (std::nothrow) Fn();
    if (!f) return fail(VKJ_ENOMEM, "vkj_module_get_function: out of host memory");
    f->mod = m;
    f->name = name;
    hipError_t e = hipModuleGetFunction(&f->fn, m->module, name);
    if (e != hipSuccess) {
        delete f;
        g_last_error = std::string("kernel '") + name + "' not found in module: " + hipGetErrorString(e);
        return (int)e;
    }
    m->functions.push_back(f);   // lives as long as its module
    *out = to_handle(f);
    return 0;
}

int vkj_buf_alloc(vkj_handle h, size_t nbytes, vkj_handle* out) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c || !out) return fail(VKJ_EINVAL, "vkj_buf_alloc: bad argument");
    if (int r = use(c)) return r;
    Buf* b = new (std::nothrow) Buf();
    if (!b) return fail(VKJ_ENOMEM, "vkj_buf_alloc: out of host memory");
    b->ctx = c;
    b->nbytes = nbytes;
    hipError_t e = hipMalloc(&b->dptr, nbytes ? nbytes : 4);
    if (e != hipSuccess) { delete b; return hip_fail(e, "hipMalloc"); }
    *out = to_handle(b);
    return 0;
}

int vkj_buf_alloc_packed(vkj_handle h, size_t nbytes, vkj_handle* out) {
    if (nbytes > PACKED_MAX_BYTES) return vkj_buf_alloc(h, nbytes, out);
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c || !out) return fail(VKJ_EINVAL, "vkj_buf_alloc_packed: bad argument");
    if (int r = use(c)) return r;
    const size_t need = ((nbytes ? nbytes : 4) + PACKED_ALIGN - 1) & ~(PACKED_ALIGN - 1);
    Slab* slab = c->slabs.empty() ? nullptr : c->slabs.back();
    if (!slab || slab->used + need > slab->size) {
        slab = new (std::nothrow) Slab();
        if (!slab) return fail(VKJ_ENOMEM, "vkj_buf_alloc_packed: out of host memory");
        hipError_t e = hipMalloc(&slab->base, SLAB_BYTES);
        if (e != hipSuccess) { delete slab; return hip_fail(e, "hipMalloc (slab)"); }
        slab->size = SLAB_BYTES;
        c->slabs.push_back(slab);
    }
    Buf* b = new (std::nothrow) Buf();
    if (!b) {
        if (slab->live == 0) { c->slabs.pop_back(); hipFree(slab->base); delete slab; }
        return fail(VKJ_ENOMEM, "vkj_buf_alloc_packed: out of host memory");
    }
    b->ctx = c;
    b->nbytes = nbytes;
    b->dptr = (char*)slab->base + slab->used;
    b->slab = slab;
    slab->used += need;
    slab->live++;
    *out = to_handle(b);
    return 0;
}

int vkj_buf_free(vkj_handle h, vkj_handle bh) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!c || !b || b->ctx != c) return fail(VKJ_EINVAL, "vkj_buf_free: bad handle");
    if (int r = use(c)) return r;
    if (b->seq_refs > 0) {
        // recorded into live sequences, which hold its address: the handle is retired now (any later
        // use of it is rejected), the memory is released when the last of those sequences is destroyed
        retire(b);
        b->released = true;
        return 0;
    }
    HIP_TRY(hipStreamSynchronize(c->stream));
    HIP_TRY(hipStreamSynchronize(c->copy_stream));
    HIP_TRY(free_buf_memory(b));
    retire(b);
    delete b;
    return 0;
}

int vkj_buf_size(vkj_handle h, vkj_handle bh, size_t* nbytes) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!c || !b || b->ctx != c || !nbytes) return fail(VKJ_EINVAL, "vkj_buf_size: bad argument");
    *nbytes = b->nbytes;
    return 0;
}

int vkj_buf_device_ptr(vkj_handle h, vkj_handle bh, uint64_t* addr) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!c || !b || b->ctx != c || !addr) return fail(VKJ_EINVAL, "vkj_buf_device_ptr: bad argument");
    *addr = (uint64_t)(uintptr_t)b->dptr;
    return 0;
}

static int check_range(const char* who, Buf* b, size_t offset, size_t nbytes) {
    if (offset > b->nbytes || nbytes > b->nbytes - offset)
        return fail(VKJ_EINVAL, "%s: range [%zu, %zu) exceeds the buffer's %zu bytes", who, offset, offset + nbytes, b->nbytes);
    return 0;
}

int vkj_buf_memset(vkj_handle h, vkj_handle bh, size_t offset, int value, size_t nbytes) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!c || !b || b->ctx != c) return fail(VKJ_EINVAL, "vkj_buf_memset: bad handle");
    if (int r = check_range("vkj_buf_memset", b, offset, nbytes)) return r;
    if (int r = use(c)) return r;
    if (nbytes) HIP_TRY(hipMemsetAsync((char*)b->dptr + offset, value, nbytes, c->stream));
    return 0;
}

int vkj_buf_upload(vkj_handle h, vkj_handle bh, size_t offset, const void* host, size_t nbytes) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!c || !b || b->ctx != c || (!host && nbytes)) return fail(VKJ_EINVAL, "vkj_buf_upload: bad argument");
    if (int r = check_range("vkj_buf_upload", b, offset, nbytes)) return r;
    if (int r = use(c)) return r;
    if (nbytes) {
        HIP_TRY(hipMemcpyAsync((char*)b->dptr + offset, host, nbytes, hipMemcpyHostToDevice, c->stream));
        HIP_TRY(hipStreamSynchronize(c->stream));
    }
    return 0;
}

int vkj_buf_download(vkj_handle h, vkj_handle bh, size_t offset, void* host, size_t nbytes) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!c || !b || b->ctx != c || (!host && nbytes)) return fail(VKJ_EINVAL, "vkj_buf_download: bad argument");
    if (int r = check_range("vkj_buf_download", b, offset, nbytes)) return r;
    if (int r = use(c)) return r;
    if (nbytes) {
        HIP_TRY(hipMemcpyAsync(host, (char*)b->dptr + offset, nbytes, hipMemcpyDeviceToHost, c->stream));
        HIP_TRY(hipStreamSynchronize(c->stream));
    }
    return 0;
}

int vkj_seq_create(vkj_handle h, int profiling, vkj_handle* out) {
    Ctx* c = from_handle<Ctx>(h, MAGIC_CTX);
    if (!c || !out) return fail(VKJ_EINVAL, "vkj_seq_create: bad argument");
    Seq* s = new (std::nothrow) Seq();
    if (!s) return fail(VKJ_ENOMEM, "vkj_seq_create: out of host memory");
    s->ctx = c;
    s->profiling = profiling != 0;
    *out = to_handle(s);
    return 0;
}

int vkj_seq_destroy(vkj_handle sh) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_destroy: bad handle");
    if (int r = use(s->ctx)) return r;
    hipStreamSynchronize(s->ctx->stream);
    hipStreamSynchronize(s->ctx->copy_stream);
    for (auto& m : s->slab_mirrors) hipHostFree(m.second);
    for (auto& t : s->uploads) {
        if (t.staging && !t.staging_mirrors_slab) hipHostFree(t.staging);
        if (t.next_staging) hipHostFree(t.next_staging);
        if (t.landing) hipFree(t.landing);
        unref_buf(t.buf);
    }
    for (auto& t : s->downloads) {
        if (t.staging) hipHostFree(t.staging);
        unref_buf(t.buf);
    }
    hipStreamSynchronize(s->ctx->side_stream);
    for (auto& l : s->launches) {
        l.fn->mod->seq_refs--;
        for (Buf* b : l.bufs) unref_buf(b);
        if (l.wait_event) hipEventDestroy(l.wait_event);
    }
    for (auto& part : s->early) {
        part.launch.fn->mod->seq_refs--;
        for (Buf* b : part.launch.bufs) unref_buf(b);
        if (part.ev_a) hipEventDestroy(part.ev_a);
        if (part.ev_b) hipEventDestroy(part.ev_b);
    }
    if (s->ev_early_done) hipEventDestroy(s->ev_early_done);
    if (s->ev_fork) hipEventDestroy(s->ev_fork);
    if (s->ev_join) hipEventDestroy(s->ev_join);
    for (auto e : s->stamps) hipEventDestroy(e);
    for (auto e : s->chunk_events) hipEventDestroy(e);
    drop_graph(s);
    retire(s);
    delete s;
    return 0;
}

static int record_transfer(const char* who, std::vector<Transfer>& list, Seq* s, vkj_handle bh,
                           size_t offset, int slot, size_t nbytes) {
    Buf* b = from_handle<Buf>(bh, MAGIC_BUF);
    if (!s || !b || b->ctx != s->ctx || slot < 0) return fail(VKJ_EINVAL, "%s: bad argument", who);
    if (int r = check_range(who, b, offset, nbytes)) return r;
    if (int r = use(s->ctx)) return r;
    Transfer t{b, offset, nbytes, slot, nullptr};
    if (nbytes && b->slab && &list == &s->uploads) {
        // staged at the array's place in a pinned copy of its slab: arrays that are neighbours in HBM are neighbours
        // there too, and one transfer can carry a run of them
        void* mirror = nullptr;
        for (auto& m : s->slab_mirrors) if (m.first == b->slab) mirror = m.second;
        if (!mirror) {
            HIP_TRY(hipHostMalloc(&mirror, b->slab->size, hipHostMallocDefault));
            s->slab_mirrors.emplace_back(b->slab, mirror);
        }
        t.staging = (char*)mirror + ((char*)b->dptr - (char*)b->slab->base) + offset;
        t.staging_mirrors_slab = true;
    } else if (nbytes) {
        HIP_TRY(hipHostMalloc(&t.staging, nbytes, hipHostMallocDefault));
    }
    list.push_back(t);
    b->seq_refs++;
    return 0;
}

int vkj_seq_record_upload(vkj_handle sh, vkj_handle bh, size_t offset, int slot, size_t nbytes) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_record_upload: bad sequence handle");
    return record_transfer("vkj_seq_record_upload", s->uploads, s, bh, offset, slot, nbytes);
}

int vkj_seq_record_download(vkj_handle sh, vkj_handle bh, size_t offset, int slot, size_t nbytes) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_record_download: bad sequence handle");
    if (int r = record_transfer("vkj_seq_record_download", s->downloads, s, bh, offset, slot, nbytes)) return r;
    // a large result comes back in chunks with an event behind each; the events are made here so
    // that an evaluation creates nothing
    if (nbytes >= STAGE_MIN)
        for (size_t off = 0; off < nbytes; off += STAGE_CHUNK) {
            hipEvent_t e;
            HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            s->chunk_events.push_back(e);
        }
    return 0;
}

// The checks and the argument block of a recorded launch (vkj_seq_record_launch, vkj_seq_record_early_part): on
// success `l` holds the launch, with the buffers' addresses patched in; nothing is referenced or recorded yet.
static int make_launch(const char* who, Seq* s, vkj_handle fh, const uint32_t grid[3], const uint32_t block[3],
                       uint32_t lds_bytes, const void* kernarg, size_t kernarg_bytes,
                       const vkj_handle* bufs, const uint32_t* buf_arg_offsets,
                       const uint64_t* buf_byte_offsets, int nbufs, Launch& l) {
    Fn*  f = from_handle<Fn>(fh, MAGIC_FN);
    if (!s || !f || f->mod->ctx != s->ctx || !grid || !block || (!kernarg && kernarg_bytes) || nbufs < 0 ||
        (nbufs && (!bufs || !buf_arg_offsets)))
        return fail(VKJ_EINVAL, "%s: bad argument", who);
    for (int i = 0; i < 3; i++)
        if (grid[i] == 0 || block[i] == 0)
            return fail(VKJ_EINVAL, "%s(%s): zero-sized grid or block", who, f->name.c_str());
    if ((uint64_t)block[0] * block[1] * block[2] > 1024)
        return fail(VKJ_EINVAL, "%s(%s): more than 1024 threads per block", who, f->name.c_str());
    if ((uint64_t)grid[0] * block[0] > 0xFFFFFFFFull || grid[1] > 65535 || grid[2] > 65535)
        return fail(VKJ_EINVAL, "%s(%s): grid too large", who, f->name.c_str());
    l.fn = f;
    for (int i = 0; i < 3; i++) { l.grid[i] = grid[i]; l.block[i] = block[i]; }
    l.lds = lds_bytes;
    l.kernarg.assign((const uint8_t*)kernarg, (const uint8_t*)kernarg + kernarg_bytes);
    for (int i = 0; i < nbufs; i++) {
        Buf* b = from_handle<Buf>(bufs[i], MAGIC_BUF);
        if (!b || b->ctx != s->ctx) return fail(VKJ_EINVAL, "%s(%s): bad buffer handle #%d", who, f->name.c_str(), i);
        uint64_t off = buf_byte_offsets ? buf_byte_offsets[i] : 0;
        if (off > b->nbytes) return fail(VKJ_EINVAL, "%s(%s): offset of buffer #%d beyond its end", who, f->name.c_str(), i);
        if (buf_arg_offsets[i] != VKJ_NO_POINTER_SLOT) {
            if ((size_t)buf_arg_offsets[i] + 8 > kernarg_bytes || (buf_arg_offsets[i] & 7))
                return fail(VKJ_EINVAL, "%s(%s): pointer slot #%d outside the argument block or misaligned", who, f->name.c_str(), i);
            uint64_t addr = (uint64_t)(uintptr_t)b->dptr + off;
            memcpy(l.kernarg.data() + buf_arg_offsets[i], &addr, 8);
        }
        l.bufs.push_back(b);
    }
    return 0;
}

int vkj_seq_record_launch(vkj_handle sh, vkj_handle fh, const uint32_t grid[3], const uint32_t block[3],
                          uint32_t lds_bytes, const void* kernarg, size_t kernarg_bytes,
                          const vkj_handle* bufs, const uint32_t* buf_arg_offsets,
                          const uint64_t* buf_byte_offsets, int nbufs) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    Launch l;
    if (int r = make_launch("vkj_seq_record_launch", s, fh, grid, block, lds_bytes, kernarg, kernarg_bytes, bufs, buf_arg_offsets,
                            buf_byte_offsets, nbufs, l)) return r;
    for (Buf* b : l.bufs) b->seq_refs++;
    l.fn->mod->seq_refs++;
    s->launches.push_back(std::move(l));
    drop_graph(s);                                  // a captured graph no longer matches the sequence
    return 0;
}

int vkj_seq_record_early_part(vkj_handle sh, vkj_handle fh, const uint32_t grid[3], const uint32_t block[3],
                              uint32_t lds_bytes, const void* kernarg, size_t kernarg_bytes,
                              const vkj_handle* bufs, const uint32_t* buf_arg_offsets,
                              const uint64_t* buf_byte_offsets, int nbufs, int upload_slot, size_t bytes_needed) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_record_early_part: bad handle");
    if (s->launches.empty()) return fail(VKJ_ESTATE, "vkj_seq_record_early_part: the launch the parts stand for is recorded first");
    const Transfer* upload = nullptr;
    for (auto& t : s->uploads) if (t.slot == upload_slot) upload = &t;
    if (!upload || bytes_needed == 0 || bytes_needed > upload->nbytes)
        return fail(VKJ_EINVAL, "vkj_seq_record_early_part: no upload in slot %d, or it has fewer than %zu bytes", upload_slot, bytes_needed);
    if (!s->early.empty() && (s->early_slot != upload_slot || bytes_needed < s->early.back().bytes_needed))
        return fail(VKJ_EINVAL, "vkj_seq_record_early_part: parts read one upload slot, in ascending order of what they need");
    if (int r = use(s->ctx)) return r;
    EarlyPart part;
    if (int r = make_launch("vkj_seq_record_early_part", s, fh, grid, block, lds_bytes, kernarg, kernarg_bytes, bufs, buf_arg_offsets,
                            buf_byte_offsets, nbufs, part.launch)) return r;
    part.bytes_needed = bytes_needed;
    // everything an evaluation needs is made here, so that evaluating creates nothing
    if (!s->ev_early_done) HIP_TRY(hipEventCreateWithFlags(&s->ev_early_done, hipEventDisableTiming));
    HIP_TRY(hipEventCreateWithFlags(&part.ev_a, hipEventDisableTiming));
    hipError_t e = hipEventCreateWithFlags(&part.ev_b, hipEventDisableTiming);
    if (e != hipSuccess) { hipEventDestroy(part.ev_a); return hip_fail(e, "hipEventCreateWithFlags"); }
    for (Buf* b : part.launch.bufs) b->seq_refs++;
    part.launch.fn->mod->seq_refs++;
    s->early_slot = upload_slot;
    s->early.push_back(std::move(part));
    return 0;
}

int vkj_seq_set_launch_lane(vkj_handle sh, int launch, int lane, int wait_for_other_lane) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_set_launch_lane: bad handle");
    if (launch < 0 || (size_t)launch >= s->launches.size() || lane < 0 || lane > 1)
        return fail(VKJ_EINVAL, "vkj_seq_set_launch_lane: launch %d of %zu, lane %d (0 or 1)", launch, s->launches.size(), lane);
    if (int r = use(s->ctx)) return r;
    Launch& l = s->launches[launch];
    // everything an evaluation needs is made here, so that evaluating creates nothing
    if (lane == 1 && !s->ev_fork) {
        HIP_TRY(hipEventCreateWithFlags(&s->ev_fork, hipEventDisableTiming | hipEventReleaseToDevice));
        hipError_t e = hipEventCreateWithFlags(&s->ev_join, hipEventDisableTiming | hipEventReleaseToDevice);
        if (e != hipSuccess) { hipEventDestroy(s->ev_fork); s->ev_fork = nullptr; return hip_fail(e, "hipEventCreateWithFlags"); }
    }
    if (wait_for_other_lane && !l.wait_event) HIP_TRY(hipEventCreateWithFlags(&l.wait_event, hipEventDisableTiming | hipEventReleaseToDevice));
    if (!wait_for_other_lane && l.wait_event) { hipEventDestroy(l.wait_event); l.wait_event = nullptr; }
    l.lane = lane;
    s->uses_side = false;
    for (auto& other : s->launches) if (other.lane) s->uses_side = true;
    drop_graph(s);
    return 0;
}

int vkj_seq_num_steps(vkj_handle sh, int* uploads, int* launches, int* downloads) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_num_steps: bad handle");
    if (uploads)   *uploads   = (int)s->uploads.size();
    if (launches)  *launches  = (int)s->launches.size();
    if (downloads) *downloads = (int)s->downloads.size();
    return 0;
}

int vkj_seq_eval(vkj_handle sh, void* const* host_ptrs, int nslots, uint32_t flags) {
    return vkj_seq_eval_next(sh, host_ptrs, nslots, flags, nullptr);
}

int vkj_seq_eval_next(vkj_handle sh, void* const* host_ptrs, int nslots, uint32_t flags, void* const* next_host_ptrs) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_eval: bad handle");
    return seq_eval(s, host_ptrs, nslots, flags, next_host_ptrs, nullptr);
}

int vkj_seq_replay(vkj_handle sh, int iters, float* ms_total) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s || iters < 1) return fail(VKJ_EINVAL, "vkj_seq_replay: bad argument");
    Ctx* c = s->ctx;
    if (int r = use(c)) return r;
    HIP_TRY(hipEventRecord(c->ev_begin, c->stream));
    for (int it = 0; it < iters; it++)
        if (int r = issue_all(c, s)) return r;
    HIP_TRY(hipEventRecord(c->ev_end, c->stream));
    HIP_TRY(hipEventSynchronize(c->ev_end));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, c->ev_begin, c->ev_end));
    if (ms_total) *ms_total = ms;
    return 0;
}

int vkj_seq_use_graph(vkj_handle sh, int enable) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_use_graph: bad handle");
    s->want_graph = enable != 0;
    if (!s->want_graph) drop_graph(s);
    return 0;
}

int vkj_seq_timestamps(vkj_handle sh, float* ms_out, int capacity, int* count) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s || !count) return fail(VKJ_EINVAL, "vkj_seq_timestamps: bad argument");
    if (!s->profiling) return fail(VKJ_ESTATE, "vkj_seq_timestamps: sequence was created without profiling");
    *count = s->stamps_valid;
    if (!ms_out) return 0;
    if (int r = use(s->ctx)) return r;
    for (int i = 0; i < s->stamps_valid && i < capacity; i++) {
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, s->stamps[0], s->stamps[i]));
        ms_out[i] = ms;
    }
    return 0;
}

}  // extern "C"
