// The parts of libvkjax_hip.so that the CPU test build of shim.cpp does not take from
// static_landing.hip (device code), and the hooks through which the test reads and steers the
// stand-in runtime.
#include "shim_internal.h"

int vkj::static_landing_init(Ctx* c) {
    static unsigned char region[VKJ_STATIC_LANDING_BYTES];
    c->static_landing = region;
    return 0;
}

// the entry point of static_landing.hip with a host copy in place of its kernel
extern "C" int vkj_seq_eval_next_static(vkj_handle sh, void* const* host_ptrs, int nslots, uint32_t flags,
                                        void* const* next_host_ptrs) {
    vkj::Seq* s = vkj::from_handle<vkj::Seq>(sh, vkj::MAGIC_SEQ);
    if (!s) return vkj::fail(VKJ_EINVAL, "vkj_seq_eval_next_static: bad handle");
    return vkj::seq_eval_static(s, host_ptrs, nslots, flags, next_host_ptrs,
                                [](void* dst, const void* src, size_t nbytes, hipStream_t) { memcpy(dst, src, nbytes); return 0; });
}

extern "C" long fake_hip_live_objects() { return (long)fake_hip().live.size(); }
extern "C" long fake_hip_creations() { return fake_hip().creations; }
extern "C" void fake_hip_on_synchronize(void (*hook)()) { fake_hip().on_synchronize = hook; }
extern "C" long fake_hip_launches() { return fake_hip().launches; }
extern "C" long fake_hip_copies() { return fake_hip().copies; }
extern "C" long fake_hip_copies_at_launch(long k) { return k >= 0 && k < (long)fake_hip().copies_at_launch.size() ? fake_hip().copies_at_launch[k] : -1; }
extern "C" void fake_hip_fail_after(long successful_calls) { fake_hip().calls_until_failure = successful_calls; }
