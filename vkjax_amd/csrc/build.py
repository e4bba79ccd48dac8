'''Build the native parts in-tree: the C-ABI runtime (libvkjax_hip.so) and the gfx950 code
objects with the kernels (one .hsaco per kernels/*.hip). Needs only hipcc; no GPU.

    python -m vkjax_amd.csrc.build [--force]
'''
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC    = os.path.dirname(os.path.abspath(__file__))
PKG     = os.path.dirname(CSRC)
ROOT    = os.path.dirname(PKG)
LIBDIR  = os.path.join(PKG, 'lib')
INCLUDE = os.path.join(ROOT, 'include')
HIPCC   = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
ARCH    = 'gfx950'

#packed fp32 instructions are switched off for all device code; no contraction of a multiply and an
#add into a fused multiply-add: every element-wise step rounds on its own, fused into another kernel or not
DEVICE_FLAGS = ['-O3', f'--offload-arch={ARCH}', '--genco', '-munsafe-fp-atomics', '-ffp-contract=off',
                '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops', '-Wno-pass-failed']

KERNEL_SOURCES = ['elementwise', 'conv_gemm', 'wgrad_gemm', 'reduce', 'index', 'threefry']


def shim_path():
    return os.path.join(LIBDIR, 'libvkjax_hip.so')


def hsaco_path(name):
    return os.path.join(LIBDIR, f'{name}.hsaco')


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f'build step failed: {" ".join(cmd)}\n{proc.stdout}')
    return proc.stdout


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def build_shim(force=True):
    '''libvkjax_hip.so = shim.cpp (host only) + static_landing.hip (the static landing array, its
    copy kernel and the entry point that allocates nothing).'''
    srcs = [os.path.join(CSRC, 'shim.cpp'), os.path.join(CSRC, 'static_landing.hip')]
    hdrs = [os.path.join(INCLUDE, 'vkjax_hip.h'), os.path.join(CSRC, 'shim_internal.h')]
    out = shim_path()
    if not force and _newer(out, srcs + hdrs):
        return out
    common = ['-O2', '-fPIC', '-pthread', '-std=c++17', f'-I{INCLUDE}', f'-I{CSRC}', '-I/opt/rocm/include']
    objs = [os.path.join(LIBDIR, 'shim.o'), os.path.join(LIBDIR, 'static_landing.o')]
    _run([HIPCC] + common + ['-x', 'c++', '-D__HIP_PLATFORM_AMD__', '-c', srcs[0], '-o', objs[0]])
    _run([HIPCC] + common + [f'--offload-arch={ARCH}', '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
                             '-c', srcs[1], '-o', objs[1]])
    _run([HIPCC, '-shared', '-pthread'] + objs + ['-o', out, '-L/opt/rocm/lib', '-lamdhip64', '-Wl,-rpath,/opt/rocm/lib'])
    for o in objs:
        os.remove(o)
    return out


def build_kernel(name, force=True):
    src  = os.path.join(CSRC, 'kernels', f'{name}.hip')
    deps = [src] + [os.path.join(CSRC, 'kernels', h) for h in ('common.h', 'ew_opcodes.h', 'ew_apply.h')]
    out  = hsaco_path(name)
    if not force and _newer(out, deps):
        return out
    _run([HIPCC] + DEVICE_FLAGS + [src, '-o', out])
    return out


def build_all(force=True, jobs=None):
    os.makedirs(LIBDIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(jobs) as pool:
        futures = [pool.submit(build_shim, force)] + [pool.submit(build_kernel, k, force) for k in KERNEL_SOURCES]
        return [f.result() for f in futures]


if __name__ == '__main__':
    for path in build_all(force='--force' in sys.argv or True):
        print('built', os.path.relpath(path, ROOT))
