// Host-only stand-in for the HIP calls that vkjax_amd/csrc/shim.cpp makes, so that the runtime's
// handle, lifetime and transfer logic can be exercised on a machine without a GPU. "Device"
// memory is host memory, every call completes before it returns, a code object is a text image
// with one kernel name per line, and the only kernel that runs is `fake_add_one`
// (arguments: uint32_t* dst, const uint32_t* src, uint32_t n -> dst[i] = src[i] + 1).
// Test infrastructure only: nothing in the package includes it.
#ifndef FAKE_HIP_RUNTIME_H
#define FAKE_HIP_RUNTIME_H

#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <set>
#include <string>
#include <vector>

typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1, hipErrorOutOfMemory = 2, hipErrorNotFound = 500, hipErrorUnknown = 999 };
enum { hipStreamNonBlocking = 1, hipEventDisableTiming = 2, hipEventReleaseToDevice = 0x40000000, hipHostMallocDefault = 0, hipStreamCaptureModeThreadLocal = 1 };
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
#define HIP_LAUNCH_PARAM_BUFFER_POINTER ((void*)1)
#define HIP_LAUNCH_PARAM_BUFFER_SIZE    ((void*)2)
#define HIP_LAUNCH_PARAM_END            ((void*)3)

struct FakeObject { int kind; };
typedef FakeObject* hipStream_t;
typedef FakeObject* hipEvent_t;
typedef FakeObject* hipGraph_t;
typedef FakeObject* hipGraphExec_t;
struct FakeModule { std::vector<std::string> kernels; };
struct FakeFunction { std::string name; };
typedef FakeModule*   hipModule_t;
typedef FakeFunction* hipFunction_t;

struct hipDeviceProp_t {
    char name[256]; char gcnArchName[256];
    int multiProcessorCount, warpSize, maxThreadsPerBlock, maxThreadsDim[3], clockRate, memoryClockRate, memoryBusWidth;
    size_t sharedMemPerBlock, totalGlobalMem;
};

// state shared with the test (exported from the test build of the shim)
struct FakeHipState {
    std::set<void*> live;          // every allocation, stream, event and module that has not been released
    long calls_until_failure = -1; // >= 0: that many further fallible calls succeed, the next one fails
    long launches = 0;
    long copies = 0;               // hipMemcpyAsync calls so far
    std::vector<long> copies_at_launch;   // per launch: how many copies had been issued before it
    long creations = 0;            // allocations (device and pinned), streams, events, modules, graphs ever made
    void (*on_synchronize)() = nullptr;   // called from inside hipStreamSynchronize (the test re-enters the library there)
};
inline FakeHipState& fake_hip() { static FakeHipState s; return s; }
inline bool fake_hip_should_fail() {
    FakeHipState& s = fake_hip();
    if (s.calls_until_failure < 0) return false;
    if (s.calls_until_failure == 0) { s.calls_until_failure = -1; return true; }
    s.calls_until_failure--;
    return false;
}
template <class T> inline hipError_t fake_hip_new(T** out) {
    if (fake_hip_should_fail()) return hipErrorOutOfMemory;
    *out = new T();
    fake_hip().creations++;
    fake_hip().live.insert(*out);
    return hipSuccess;
}
template <class T> inline hipError_t fake_hip_delete(T* p) {
    if (!fake_hip().live.erase(p)) return hipErrorInvalidValue;
    delete p;
    return hipSuccess;
}

inline const char* hipGetErrorString(hipError_t e) { return e == hipErrorOutOfMemory ? "out of memory (injected)" : e == hipSuccess ? "no error" : "fake hip error"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
inline hipError_t hipSetDevice(int) { return hipSuccess; }
inline hipError_t hipGetDeviceProperties(hipDeviceProp_t* p, int) {
    memset(p, 0, sizeof(*p));
    strcpy(p->name, "fake"); strcpy(p->gcnArchName, "gfx950");
    p->multiProcessorCount = 256; p->warpSize = 64; p->maxThreadsPerBlock = 1024; p->maxThreadsDim[0] = 1024;
    return hipSuccess;
}
inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { return fake_hip_new(s); }
inline hipError_t hipStreamDestroy(hipStream_t s) { return fake_hip_delete(s); }
inline hipError_t hipStreamSynchronize(hipStream_t) {
    if (auto hook = fake_hip().on_synchronize) { fake_hip().on_synchronize = nullptr; hook(); }
    return hipSuccess;
}
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t* e) { return fake_hip_new(e); }
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { return fake_hip_new(e); }
inline hipError_t hipEventDestroy(hipEvent_t e) { return fake_hip_delete(e); }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 0.f; return hipSuccess; }
inline hipError_t fake_hip_alloc(void** p, size_t n) {
    if (fake_hip_should_fail()) return hipErrorOutOfMemory;
    *p = malloc(n ? n : 1);
    memset(*p, 0xCD, n ? n : 1);           // never hand out zeroed memory: stale-data bugs must show
    fake_hip().creations++;
    fake_hip().live.insert(*p);
    return hipSuccess;
}
inline hipError_t fake_hip_release(void* p) {
    if (!fake_hip().live.erase(p)) return hipErrorInvalidValue;
    free(p);
    return hipSuccess;
}
inline hipError_t hipMalloc(void** p, size_t n) { return fake_hip_alloc(p, n); }
inline hipError_t hipFree(void* p) { return fake_hip_release(p); }
inline hipError_t hipHostMalloc(void** p, size_t n, unsigned) { return fake_hip_alloc(p, n); }
inline hipError_t hipHostFree(void* p) { return fake_hip_release(p); }
inline hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, hipMemcpyKind, hipStream_t) { fake_hip().copies++; memmove(dst, src, n); return hipSuccess; }
inline hipError_t hipMemsetAsync(void* dst, int v, size_t n, hipStream_t) { memset(dst, v, n); return hipSuccess; }
inline hipError_t hipModuleLoadData(hipModule_t* m, const void* image) {
    if (hipError_t e = fake_hip_new(m)) return e;
    std::string text((const char*)image), name;
    for (char ch : text + "\n") {
        if (ch == '\n') { if (!name.empty()) (*m)->kernels.push_back(name); name.clear(); }
        else name += ch;
    }
    return hipSuccess;
}
inline hipError_t hipModuleUnload(hipModule_t m) { return fake_hip_delete(m); }
inline hipError_t hipModuleGetFunction(hipFunction_t* f, hipModule_t m, const char* name) {
    for (auto& k : m->kernels)
        if (k == name) { *f = new FakeFunction{k}; return hipSuccess; }     // owned by nobody, like a real hipFunction_t
    return hipErrorNotFound;
}
inline hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned,
                                        unsigned, hipStream_t, void**, void** extra) {
    fake_hip().launches++;
    fake_hip().copies_at_launch.push_back(fake_hip().copies);
    if (f->name != "fake_add_one") return hipSuccess;
    struct Args { uint32_t* dst; const uint32_t* src; uint32_t n; } a;
    memcpy(&a, extra[1], sizeof(a));
    for (uint32_t i = 0; i < a.n; i++) a.dst[i] = a.src[i] + 1u;
    return hipSuccess;
}
// graphs are not imitated: capture fails, and the runtime falls back to individual launches
inline hipError_t hipStreamBeginCapture(hipStream_t, int) { return hipErrorUnknown; }
inline hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t*) { return hipErrorUnknown; }
inline hipError_t hipGraphInstantiate(hipGraphExec_t*, hipGraph_t, void*, void*, size_t) { return hipErrorUnknown; }
inline hipError_t hipGraphDestroy(hipGraph_t) { return hipSuccess; }
inline hipError_t hipGraphExecDestroy(hipGraphExec_t) { return hipSuccess; }
inline hipError_t hipGraphLaunch(hipGraphExec_t, hipStream_t) { return hipErrorUnknown; }

#endif
