// The parts of libvkjax_hip.so that the CPU test build of shim.cpp does not take from
// static_landing.hip (device code), and the hooks through which the test reads and steers the
// stand-in runtime.
#include "shim_internal.h"

int vkj::static_landing_init(Ctx* c) {
    static unsigned char region[1 << 16];
    c->static_landing = region;
    return 0;
}

extern "C" long fake_hip_live_objects() { return (long)fake_hip().live.size(); }
extern "C" long fake_hip_launches() { return fake_hip().launches; }
extern "C" void fake_hip_fail_after(long successful_calls) { fake_hip().calls_until_failure = successful_calls; }
