// Objects behind the handles of include/vkjax_hip.h, shared by the translation units of
// libvkjax_hip.so (shim.cpp: the runtime; static_landing.hip: the entry point that allocates
// nothing). Not part of the C ABI.
#ifndef VKJAX_SHIM_INTERNAL_H
#define VKJAX_SHIM_INTERNAL_H

#include "vkjax_hip.h"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace vkj {

int fail(int code, const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define HIP_TRY(expr)                                          \
    do {                                                       \
        hipError_t _e = (expr);                                \
        if (_e != hipSuccess) return ::vkj::hip_fail(_e, #expr); \
    } while (0)

constexpr uint32_t MAGIC_CTX = 0x766b4a43, MAGIC_BUF = 0x766b4a42, MAGIC_MOD = 0x766b4a4d,
                   MAGIC_FN = 0x766b4a46, MAGIC_SEQ = 0x766b4a53;

// Small arrays that travel together (a network's per-feature vectors) are carved out of slabs, one next to the other
// at 256-byte steps (vkj_buf_alloc_packed), so that an evaluation can send a run of them with one transfer. A slab
// goes when the last array carved from it has gone; space is not handed out twice.
struct Slab {
    void*  base = nullptr;
    size_t size = 0, used = 0;
    int    live = 0;
};
constexpr size_t SLAB_BYTES = 1u << 20, PACKED_MAX_BYTES = 64u << 10, PACKED_ALIGN = 256;

struct Ctx {
    uint64_t    handle = 0;
    uint32_t    magic = MAGIC_CTX;
    int         device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t  ev_begin = nullptr, ev_end = nullptr;
    hipStream_t copy_stream = nullptr;   // uploads that overlap the launches of `stream`
    hipStream_t side_stream = nullptr;   // launches of lane 1: work that does not depend on what `stream` is running
    hipEvent_t  ev_landed = nullptr;     // the following evaluation's arguments have reached HBM
    hipEvent_t  ev_uploaded = nullptr;   // this evaluation's own uploads have left their staging buffers
    hipEvent_t  ev_copied = nullptr;     // the share of this evaluation's uploads that went over the second stream has arrived
    // Launches that follow the uploads (seq_eval): the chunks then alternate between copy_stream and side_stream, and
    // at each of a few checkpoints along the upload the launch stream is told to wait for what both have been handed
    // so far (one event per copy stream and checkpoint), before the launches that need no more than that are issued.
    // (No further stream for this: a process has few hardware queues, streams are dealt out over them in turn, and
    // with three streams per context the launch streams of up to four contexts end up on different queues - which is
    // what lets the lanes of Function.stream(in_flight=...) run side by side. With four they all shared one.)
    static constexpr int MAX_CHECKPOINTS = 8;
    hipEvent_t  ev_checkpoint[2 * MAX_CHECKPOINTS] = {};
    std::vector<Slab*> slabs;            // those with live arrays; the last one is the one being filled
    void*       static_landing = nullptr;   // this device's copy of the static landing array (static_landing.hip)
};

// A buffer recorded into sequences stays allocated until the last of them is destroyed:
// vkj_buf_free on such a buffer retires the handle at once and defers the release.
struct Buf {
    uint64_t handle = 0;
    uint32_t magic = MAGIC_BUF;
    Ctx*     ctx = nullptr;
    void*    dptr = nullptr;
    size_t   nbytes = 0;
    int      seq_refs = 0;       // recorded transfers and launch arguments of live sequences
    bool     released = false;   // vkj_buf_free was called; memory goes when seq_refs drops to 0
    Slab*    slab = nullptr;     // the slab `dptr` points into (vkj_buf_alloc_packed), or null: an allocation of its own
};

struct Fn;
struct Mod {
    uint64_t         handle = 0;
    uint32_t         magic = MAGIC_MOD;
    Ctx*             ctx = nullptr;
    hipModule_t      module = nullptr;
    int              seq_refs = 0;   // recorded launches of live sequences; unloading is refused while > 0
    std::vector<Fn*> functions;      // retired and deleted together with the module
};

struct Fn {
    uint64_t      handle = 0;
    uint32_t      magic = MAGIC_FN;
    Mod*          mod = nullptr;
    hipFunction_t fn = nullptr;
    std::string   name;
};

struct Transfer {
    Buf*   buf;
    size_t offset, nbytes;
    int    slot;
    void*  staging;                  // pinned host memory owned by the sequence
    bool   staging_mirrors_slab = false;   // ... inside the sequence's pinned copy of the buffer's slab, at the buffer's place in it
    void*  next_staging = nullptr;   // pinned host memory and device memory for the arguments of the
    void*  landing = nullptr;        // following evaluation, allocated when one is first handed in
};

struct Launch {
    Fn*                  fn;
    uint32_t             grid[3], block[3], lds;
    std::vector<uint8_t> kernarg;
    std::vector<Buf*>    bufs;       // the buffers whose addresses the argument block holds
    int                  lane = 0;   // 0: the context's stream, 1: its side stream
    hipEvent_t           wait_event = nullptr;   // made when the launch is told to wait for the other lane: recorded there
                                                 // and waited for on this launch's lane before the launch is issued
};

// One part of the first launch's alternative form (vkj_seq_record_early_part): what it needs of the argument in
// upload slot Seq::early_slot, and the two events that tell its stream that those bytes have arrived.
struct EarlyPart {
    Launch     launch;
    size_t     bytes_needed = 0;
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
};

struct Seq {
    uint64_t                handle = 0;
    uint32_t                magic = MAGIC_SEQ;
    Ctx*                    ctx = nullptr;
    bool                    profiling = false;
    std::vector<Transfer>   uploads, downloads;
    std::vector<Launch>     launches;
    std::vector<hipEvent_t> chunk_events;   // one behind every chunk of a large download
    std::vector<hipEvent_t> stamps;         // profiling: 1 + number of steps
    int                     stamps_valid = 0;
    bool                    uses_side = false;      // some launch is on lane 1
    hipEvent_t              ev_fork = nullptr;      // lane 1 starts behind everything queued on the stream so far (uploads)
    hipEvent_t              ev_join = nullptr;      // the stream continues (downloads, the final wait) behind lane 1
    bool                    want_graph = false;     // issue the launches as one captured graph
    bool                    graph_failed = false;   // capture did not work once: keep to plain launches
    hipGraphExec_t          graph_exec = nullptr;
    std::vector<std::pair<Slab*, void*>> slab_mirrors;   // pinned memory laid out like a slab: the staging of the uploads into its arrays
    std::vector<EarlyPart>  early;                  // the first launch in parts, each issued while the rest of an argument is still on its way
    int                     early_slot = -1;
    hipEvent_t              ev_early_done = nullptr;
};

// Handles are keys into a process-wide table, never raw addresses, so that a stale or made-up
// handle is rejected instead of being dereferenced.
struct Registry {
    std::mutex mu;
    std::unordered_map<uint64_t, std::pair<uint32_t, void*>> live;
    uint64_t next = 0x1000;
};
Registry& registry();

template <class T>
T* from_handle(vkj_handle h, uint32_t magic) {
    Registry& r = registry();
    std::lock_guard<std::mutex> lock(r.mu);
    auto it = r.live.find(h);
    if (it == r.live.end() || it->second.first != magic) return nullptr;
    return static_cast<T*>(it->second.second);
}
template <class T>
vkj_handle to_handle(T* p) {
    Registry& r = registry();
    std::lock_guard<std::mutex> lock(r.mu);
    const uint64_t h = r.next++;
    r.live[h] = {p->magic, p};
    p->handle = h;
    return h;
}
template <class T>
void retire(T* p) {
    Registry& r = registry();
    std::lock_guard<std::mutex> lock(r.mu);
    r.live.erase(p->handle);
}

// Where the arguments of the following evaluation wait in HBM until this evaluation's launches
// are through. The default (null) is one hipMalloc per upload slot on first use, pinned staging
// of its own, and device-to-device copies; the static variant hands in a fixed region and a
// kernel launch that moves its contents on.
struct LandingRegion {
    char*  base;       // device address of the region
    size_t capacity;   // bytes
    // copies nbytes from src (inside the region) to dst on `stream`
    int (*move)(void* dst, const void* src, size_t nbytes, hipStream_t stream);
};

int seq_eval(Seq* s, void* const* host_ptrs, int nslots, uint32_t flags, void* const* next_host_ptrs,
             const LandingRegion* region);

// vkj_seq_eval_next_static without its handle lookup: refuses what would make the evaluation allocate
// (time stamps, a graph that is not built yet), arguments beyond the array's size and a call that overlaps
// another one on the same GPU, then evaluates with the context's static landing array and `move`.
int seq_eval_static(Seq* s, void* const* host_ptrs, int nslots, uint32_t flags, void* const* next_host_ptrs,
                    int (*move)(void* dst, const void* src, size_t nbytes, hipStream_t stream));

// static_landing.hip: resolves the device address of the static landing array for the current device
int static_landing_init(Ctx* c);

}  // namespace vkj

#endif
