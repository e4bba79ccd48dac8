/*
 * vkjax_hip.h - C ABI of the MI355X device runtime behind vkJAX's jaxpr interpreter.
 *
 * This library takes the place of the Vulkan-Kompute objects the reference drives from
 * Python (kp.Manager / kp.Tensor / kp.Sequence / kp.OpAlgoDispatch / kp.OpTensorSync*,
 * package kp==0.7.0): a device context, HBM buffers, gfx950 code objects and a recorded
 * sequence of uploads, kernel launches and downloads that is replayed with ONE call per
 * run. All work of a context is issued on one in-order HIP stream (vkj_seq_eval_next adds
 * a second one that only carries the following call's uploads); nothing synchronises
 * with the host except the tail of vkj_seq_eval / vkj_seq_eval_next / vkj_seq_replay, the
 * blocking buffer transfers and vkj_sync.
 *
 * Conventions: every function returns 0 on success, a positive hipError_t or a negative
 * VKJ_E* code otherwise; vkj_last_error() returns the message of the calling thread's last
 * failure. Handles are opaque 64-bit values owned by the library. Host memory passed in is
 * owned by the caller and only has to stay valid for the duration of the call. A context
 * and its objects must be used from one thread at a time.
 */
#ifndef VKJAX_HIP_H
#define VKJAX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t vkj_handle;

enum {
    VKJ_EINVAL   = -1,   /* bad argument (null pointer, out-of-range size, unknown handle) */
    VKJ_ENOMEM   = -2,
    VKJ_ESTATE   = -3,   /* call not valid in the object's current state */
    VKJ_ENODEV   = -4    /* no usable GPU */
};

/* vkj_seq_eval flags */
enum {
    VKJ_EVAL_DEFAULT        = 0,
    VKJ_EVAL_SKIP_UPLOADS   = 1,   /* inputs are already resident in HBM */
    VKJ_EVAL_SKIP_DOWNLOADS = 2,
    VKJ_EVAL_NULL_IS_RESIDENT = 4  /* an upload slot whose host pointer is NULL is skipped: its buffer keeps what it holds */
};

typedef struct vkj_props {
    char     name[256];
    char     arch[64];                 /* e.g. "gfx950:sramecc+:xnack-" */
    int32_t  compute_units;
    int32_t  wavefront_size;
    int32_t  max_threads_per_block;    /* replaces max_work_group_invocations */
    int32_t  max_block_dim_x;          /* replaces max_work_group_size[0] */
    int32_t  lds_bytes_per_block;
    int32_t  clock_khz;
    int32_t  memory_clock_khz;
    int32_t  memory_bus_bits;
    uint64_t hbm_bytes;
} vkj_props;

const char* vkj_last_error(void);
int vkj_device_count(int* count);

/* kp.Manager(device_index)            reference: vkjax/kompute_jaxpr_interpreter.py:19-20 */
int vkj_ctx_create(int device, vkj_handle* ctx);
int vkj_ctx_destroy(vkj_handle ctx);
/* mgr.get_device_properties()         reference: vkjax/kompute_jaxpr_interpreter.py:100-102 */
int vkj_device_props(vkj_handle ctx, vkj_props* out);
/* blocks until everything issued on the context's stream has finished */
int vkj_sync(vkj_handle ctx);

/* Code objects built ahead of time for gfx950 replace the per-op SPIR-V produced by
 * pyshaderc.compile_into_spirv          reference: vkjax/shaders.py:16-29 */
int vkj_module_load(vkj_handle ctx, const void* image, size_t nbytes, vkj_handle* module);
/* Unloading retires the module's function handles with it. A module that recorded launches of
 * live sequences refer to is not unloaded: VKJ_ESTATE until those sequences are destroyed. */
int vkj_module_unload(vkj_handle ctx, vkj_handle module);
int vkj_module_get_function(vkj_handle ctx, vkj_handle module, const char* name, vkj_handle* function);

/* mgr.tensor(array) + OpTensorSyncDevice  reference: vkjax/buffers.py:189-204 */
int vkj_buf_alloc(vkj_handle ctx, size_t nbytes, vkj_handle* buf);
/* The handle is retired at once. The memory of a buffer that live sequences have recorded (they hold
 * its address) is released when the last of those sequences is destroyed. */
/* The same for arrays that are uploaded together, call after call (the parameter vectors of a network: hundreds of
 * arrays of a few KB): arrays of at most 64 KB are placed next to each other, 256 bytes apart at least, in slabs of
 * 1 MB, and a sequence stages its uploads into them side by side as well, so that an evaluation sends a run of
 * neighbours with one transfer instead of one each. Larger requests are served as by vkj_buf_alloc. A buffer is
 * used and freed like any other; a slab's memory is returned when the last buffer in it is freed.
 *                                     reference: mgr.tensor(...) per variable, vkjax/buffers.py:202 */
int vkj_buf_alloc_packed(vkj_handle ctx, size_t nbytes, vkj_handle* buf);
int vkj_buf_free(vkj_handle ctx, vkj_handle buf);
int vkj_buf_size(vkj_handle ctx, vkj_handle buf, size_t* nbytes);
int vkj_buf_device_ptr(vkj_handle ctx, vkj_handle buf, uint64_t* device_address);
int vkj_buf_memset(vkj_handle ctx, vkj_handle buf, size_t offset, int byte_value, size_t nbytes);
/* blocking host->device / device->host copies (build-time constants, debugging reads:
 * tensor.data(), OpTensorSyncLocal on all tensors  reference: vkjax/kompute_jaxpr_interpreter.py:85-89) */
int vkj_buf_upload(vkj_handle ctx, vkj_handle buf, size_t offset, const void* host, size_t nbytes);
int vkj_buf_download(vkj_handle ctx, vkj_handle buf, size_t offset, void* host, size_t nbytes);

/* mgr.sequence(total_timestamps=n)    reference: vkjax/kompute_jaxpr_interpreter.py:48-49
 * profiling != 0 records one timestamp before the first step and one after every step. */
int vkj_seq_create(vkj_handle ctx, int profiling, vkj_handle* seq);
int vkj_seq_destroy(vkj_handle seq);
/* seq.record(kp.OpTensorSyncDevice([...]))  reference: vkjax/kompute_jaxpr_interpreter.py:51-53
 * `slot` indexes the host_ptrs array given to vkj_seq_eval. */
int vkj_seq_record_upload(vkj_handle seq, vkj_handle buf, size_t offset, int slot, size_t nbytes);
/* mgr.algorithm(tensors, spirv, workgroup) + seq.record(kp.OpAlgoDispatch(algo))
 *                                     reference: vkjax/kompute_jaxpr_interpreter.py:55-60
 * `kernarg` is the kernel's argument block laid out by the caller. For each i < nbufs the
 * 8 bytes at kernarg[buf_arg_offsets[i]] are overwritten with the device address of
 * bufs[i] plus buf_byte_offsets[i] (may be NULL for all-zero). Addresses are resolved
 * once, here. A buffer with buf_arg_offsets[i] == VKJ_NO_POINTER_SLOT gets no address written: the
 * kernel reaches it through addresses it finds elsewhere (a table in device memory); the sequence
 * keeps it alive like the others. Every buffer the kernel reads must be listed in one of the two
 * ways: an evaluation that uploads large arguments sends them in the order in which the launches
 * first read them and issues each launch as soon as what it and the launches before it read has
 * been handed to the copy engines, while later arguments are still on their way (the reference
 * uploads everything, then evaluates: vkjax/kompute_jaxpr_interpreter.py:72-77). */
#define VKJ_NO_POINTER_SLOT 0xFFFFFFFFu
int vkj_seq_record_launch(vkj_handle seq, vkj_handle function,
                          const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes,
                          const void* kernarg, size_t kernarg_bytes,
                          const vkj_handle* bufs, const uint32_t* buf_arg_offsets,
                          const uint64_t* buf_byte_offsets, int nbufs);
/* seq.record(kp.OpTensorSyncLocal([...]))   reference: vkjax/kompute_jaxpr_interpreter.py:62-63 */
int vkj_seq_record_download(vkj_handle seq, vkj_handle buf, size_t offset, int slot, size_t nbytes);
/* There is no vkj_seq_record_memset: an array that has to start at zero inside a sequence (the table
 * a scatter-add accumulates into) is cleared by a recorded launch of the fill kernel. hipMemsetAsync
 * nodes inside a captured graph have given wrong results on replays after the first, and
 * vkj_seq_use_graph captures the launches of a sequence. vkj_buf_memset clears a buffer outside
 * sequences. */
/* Puts recorded launch number `launch` (0-based, in recording order) on lane 0 (the context's stream, the
 * default) or lane 1 (a second stream of the same priority), and says whether its lane has to wait, before
 * the launch is issued, for everything recorded before it on the OTHER lane. Launches keep their recorded
 * order within a lane; lane 1 starts behind the uploads and is joined before the downloads. The caller
 * is responsible for the waits its data dependencies need (read after write, write after read and write
 * after write, on the memory the launches touch). Events are created here, none when evaluating. A
 * sequence replayed as a graph or created with timestamps issues all launches on lane 0 in recorded
 * order. The reference records every dispatch into one in-order sequence
 * (vkjax/kompute_jaxpr_interpreter.py:55-60); this lets launches that do not depend on each other share
 * the GPU (the index passes of a scatter-add beside a gather, a projection beside the branch it joins). */
int vkj_seq_set_launch_lane(vkj_handle seq, int launch, int lane, int wait_for_other_lane);
/* An alternative form of the FIRST recorded launch, for evaluations that upload the argument in `upload_slot`: the
 * launch cut into parts (recorded with one call each, in order; arguments as for vkj_seq_record_launch) that
 * together compute exactly what it computes, part k reading no more than the first `bytes_needed` bytes of that
 * argument (ascending over the parts). When an evaluation sends that argument as the last one of its chunked
 * uploads (VKJ uploads of 8 MB and more travel in chunks), each part is issued, on a stream of its own, as soon as
 * the chunks it reads have been handed to the copy engines, so the device computes while the rest of the argument
 * is still on its way; the first launch itself is then skipped and the others follow the last part. In every other
 * evaluation (the argument resident or small, time stamps, a captured graph, launches on two lanes) the first launch
 * runs as recorded. Events are created here, none when evaluating. The reference uploads every argument, then
 * evaluates (vkjax/kompute_jaxpr_interpreter.py:72-77). */
int vkj_seq_record_early_part(vkj_handle seq, vkj_handle fn, const uint32_t grid[3], const uint32_t block[3],
                              uint32_t lds_bytes, const void* kernarg, size_t kernarg_bytes,
                              const vkj_handle* bufs, const uint32_t* buf_arg_offsets,
                              const uint64_t* buf_byte_offsets, int nbufs, int upload_slot, size_t bytes_needed);
int vkj_seq_num_steps(vkj_handle seq, int* uploads, int* launches, int* downloads);
/* sequence.eval()                     reference: vkjax/kompute_jaxpr_interpreter.py:77
 * All uploads, then all launches, then all downloads, then one stream synchronisation.
 * host_ptrs[slot] supplies the host address of every recorded upload and download. */
int vkj_seq_eval(vkj_handle seq, void* const* host_ptrs, int nslots, uint32_t flags);
/* vkj_seq_eval that also brings in the arguments of the FOLLOWING evaluation while the device runs
 * this one's launches: every upload slot whose next_host_ptrs entry is not NULL is staged and sent,
 * on a second stream, to a landing buffer in HBM (allocated on first use, one per such slot), and
 * copied on into its argument buffer once this evaluation's launches are through. The following
 * call then passes NULL for those slots with VKJ_EVAL_NULL_IS_RESIDENT. next_host_ptrs has nslots
 * entries or is NULL (then the call is vkj_seq_eval). The reference copies and runs strictly in
 * turn (vkjax/kompute_jaxpr_interpreter.py:72-77); this is the overlap of the two. */
int vkj_seq_eval_next(vkj_handle seq, void* const* host_ptrs, int nslots, uint32_t flags,
                      void* const* next_host_ptrs);
/* vkj_seq_eval_next that allocates nothing. No counterpart in the reference; it is for callers that
 * cannot allocate device or pinned memory where they evaluate (serving loops, harnesses that
 * forbid hipMalloc): the following evaluation's arguments land in an array of
 * VKJ_STATIC_LANDING_BYTES that is part of the library's device image (every GPU the library runs
 * on holds one copy until the process ends), are staged in the pinned buffers the sequence already
 * owns, and are moved on by a copy kernel. Slots are packed at multiples of 256 bytes; arguments
 * that do not fit are rejected with VKJ_EINVAL, sequences with timestamps, or with a graph that is
 * not built yet, with VKJ_ESTATE. All calls on one GPU share the array, which a call claims until it
 * returns: a call that overlaps another one on the same GPU (another thread or context) is rejected
 * with VKJ_ESTATE ("static landing array busy") and may be repeated. Same arguments and results as
 * vkj_seq_eval_next otherwise. */
#define VKJ_STATIC_LANDING_BYTES (64u << 20)
int vkj_seq_eval_next_static(vkj_handle seq, void* const* host_ptrs, int nslots, uint32_t flags,
                             void* const* next_host_ptrs);
/* Launches only, `iters` times back to back, bracketed by two events on the context's
 * stream; *ms_total receives the elapsed device time of all iterations. Used for
 * measurement with inputs resident in HBM. No counterpart in the reference. */
int vkj_seq_replay(vkj_handle seq, int iters, float* ms_total);
/* Makes vkj_seq_eval and vkj_seq_replay issue the launches of this sequence as ONE captured HIP
 * graph (built at the next use, rebuilt after further recording) instead of one launch call
 * each; uploads, downloads and profiling events stay outside the graph. enable = 0 returns to
 * individual launches. A sequence created with timestamps never uses a graph. The counterpart
 * in the reference is the Vulkan command buffer the sequence is recorded into once
 * (vkjax/kompute_jaxpr_interpreter.py:49-63). */
int vkj_seq_use_graph(vkj_handle seq, int enable);
/* sequence.get_timestamps()           reference: vkjax/kompute_jaxpr_interpreter.py:91-95
 * Milliseconds since the first timestamp of the last vkj_seq_eval; *count receives the
 * number of timestamps available (steps + 1). */
int vkj_seq_timestamps(vkj_handle seq, float* ms_out, int capacity, int* count);

#ifdef __cplusplus
}
#endif
#endif /* VKJAX_HIP_H */
