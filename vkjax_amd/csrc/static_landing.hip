// vkj_seq_eval_next_static: vkj_seq_eval_next for callers that must not allocate (serving loops
// and harnesses in which hipMalloc is forbidden or too slow to tolerate on the request path).
//
// vkj_seq_eval_next parks the arguments of the following evaluation in landing buffers in HBM
// that it allocates, with pinned staging memory of their own, when a slot is first handed in.
// Here the landing buffers are pieces of one array that is part of the library's device image,
// the pinned buffer every recorded upload already owns serves as staging, and a copy kernel
// moves the landed arguments on. Streams and events are made by vkj_ctx_create. The entry point
// therefore calls no hipMalloc, hipHostMalloc, hipFree, stream or event creation.
//
// Every GPU the library runs on holds its own copy of the array (VKJ_STATIC_LANDING_BYTES) from
// the moment the library is loaded there until the process ends. All calls on one GPU share it,
// and it keeps what the last call left: a call only reads back the bytes it has just written,
// so nothing needs clearing. Two calls that overlap in time on one GPU (two threads, two
// contexts) would race on it: the array is claimed for the duration of a call and the second
// caller is refused with VKJ_ESTATE (seq_eval_static in shim.cpp, which also holds the other
// refusals, so that the host-only test build exercises them).
#include "shim_internal.h"

#include <cstring>

using namespace vkj;

static __device__ __align__(256) unsigned char scratch[VKJ_STATIC_LANDING_BYTES];

namespace {

// dst[0 .. nbytes) = src[0 .. nbytes); 16 bytes per lane where both sides allow it
__global__ __launch_bounds__(256) void move_landed(unsigned char* __restrict__ dst, const unsigned char* __restrict__ src,
                                                   size_t nbytes, int vectors) {
    const size_t stride = (size_t)gridDim.x * 256u;
    size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (vectors) {
        const size_t nvec = nbytes / 16u;
        const uint4* s4 = reinterpret_cast<const uint4*>(src);
        uint4* d4 = reinterpret_cast<uint4*>(dst);
        for (size_t v = i; v < nvec; v += stride) d4[v] = s4[v];
        for (size_t b = nvec * 16u + i; b < nbytes; b += stride) dst[b] = src[b];
    } else {
        for (; i < nbytes; i += stride) dst[i] = src[i];
    }
}

int move_on(void* dst, const void* src, size_t nbytes, hipStream_t stream) {
    if (!nbytes) return 0;
    const int vectors = (((uintptr_t)dst | (uintptr_t)src) & 15u) == 0;
    const size_t items = vectors ? (nbytes + 15u) / 16u : nbytes;
    size_t blocks = (items + 255u) / 256u;
    if (blocks > 8192u) blocks = 8192u;              // 32 workgroups per CU; the kernel strides over the rest
    // launched through the call that returns its own status: hipGetLastError would also hand back what an
    // earlier, unrelated call left behind (a kernel name looked up in the wrong module)
    unsigned char* d = (unsigned char*)dst;
    const unsigned char* s = (const unsigned char*)src;
    int vec = vectors;
    void* args[] = {&d, &s, &nbytes, &vec};
    HIP_TRY(hipLaunchKernel((const void*)move_landed, dim3((unsigned)blocks), dim3(256), args, 0, stream));
    return 0;
}

}  // namespace

// Called by vkj_ctx_create with the context's device current: the array's name is only a
// host-side stand-in, its address on this device has to be asked for.
int vkj::static_landing_init(Ctx* c) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(VKJ_ENODEV, "vkj_ctx_create: the static landing array has no address on device %d", c->device);
    c->static_landing = p;
    return 0;
}

extern "C" int vkj_seq_eval_next_static(vkj_handle sh, void* const* host_ptrs, int nslots, uint32_t flags,
                                        void* const* next_host_ptrs) {
    Seq* s = from_handle<Seq>(sh, MAGIC_SEQ);
    if (!s) return fail(VKJ_EINVAL, "vkj_seq_eval_next_static: bad handle");
    return seq_eval_static(s, host_ptrs, nslots, flags, next_host_ptrs, move_on);
}
