"""Builds the native artefacts of the package for gfx950, in-tree:

  deep_ep/lib/ep_kernels.hsaco     device code object   (hipcc --genco)
  deep_ep/lib/libdeep_ep_hip.so    host runtime, C ABI  (hipcc -shared)
  deep_ep/_native.*.so             compiled Python binding of dispatch/combine over that C ABI  (g++, pybind11 + torch headers)
  deep_ep/lib/abi_client           a plain-C caller of the C ABI, used by the tests  (gcc)
  ep_calib/lib/ep_calib.hsaco      calibration kernels of the benchmarks (not part of the product)
  ep_calib/lib/libdeep_ep_calib.so their host side, C ABI of include/deep_ep_calib.h

hipcc cross-compiles, so this runs on a machine without a GPU.  `python deepep-ascend_amd/deep_ep/_build.py`.
"""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(PKG), 'csrc')
LIB = os.path.join(PKG, 'lib')
CALIB_LIB = os.path.join(os.path.dirname(PKG), 'ep_calib', 'lib')
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')

DEVICE_FLAGS = [
    '--offload-arch=gfx950', '--genco', '-O3', '-std=c++17',
    '-ffp-contract=off',                              # combine and quantiser round every product and sum
    '-fhip-fp32-correctly-rounded-divide-sqrt',       # 448/amax and amax/448 are IEEE divisions
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
]
# the runtime is compiled as HIP: it holds one device array (the static scratch of ep_dispatch_static_launch)
HOST_FLAGS = ['-x', 'hip', '--offload-arch=gfx950', '-shared', '-fPIC', '-O2', '-std=c++17', '-Wall',
              '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']
ROCM = os.environ.get('ROCM_PATH', '/opt/rocm')
C_CLIENT_FLAGS = ['-std=c11', '-O1', '-Wall', '-D__HIP_PLATFORM_AMD__', f'-I{ROCM}/include']


def binding_command():
    """g++ line of the compiled binding: torch's headers and libraries (ROCm build), its bundled pybind11."""
    import sysconfig
    import torch
    tdir = os.path.dirname(torch.__file__)
    inc, tlib = os.path.join(tdir, 'include'), os.path.join(tdir, 'lib')
    out = os.path.join(PKG, '_native' + sysconfig.get_config_var('EXT_SUFFIX'))
    return ['g++', '-O2', '-std=c++17', '-shared', '-fPIC', '-fvisibility=hidden', '-Wall', '-Wno-unused-function',
            f'-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}', '-DUSE_ROCM', '-D__HIP_PLATFORM_AMD__=1',
            f'-I{inc}', f'-I{inc}/torch/csrc/api/include', f'-I{ROCM}/include', f'-I{sysconfig.get_paths()["include"]}',
            os.path.join(CSRC, 'python_api.cpp'), '-o', out,
            f'-L{LIB}', '-ldeep_ep_hip', f'-L{tlib}', '-ltorch_python', '-ltorch', '-ltorch_cpu', '-ltorch_hip', '-lc10', '-lc10_hip',
            '-Wl,-rpath,$ORIGIN/lib', f'-Wl,-rpath,{tlib}']


def run(cmd):
    print(' '.join(cmd), flush=True)
    subprocess.check_call(cmd)


def build(verbose: bool = True) -> None:
    os.makedirs(LIB, exist_ok=True)
    run([HIPCC, *DEVICE_FLAGS, '-o', os.path.join(LIB, 'ep_kernels.hsaco'), os.path.join(CSRC, 'ep_kernels.hip')])
    run([HIPCC, *HOST_FLAGS, '-o', os.path.join(LIB, 'libdeep_ep_hip.so'), os.path.join(CSRC, 'ep_runtime.cpp')])
    run(binding_command())
    os.makedirs(CALIB_LIB, exist_ok=True)
    run([HIPCC, *DEVICE_FLAGS, '-o', os.path.join(CALIB_LIB, 'ep_calib.hsaco'), os.path.join(CSRC, 'ep_calib.hip')])
    run([HIPCC, '-shared', '-fPIC', '-O2', '-std=c++17', '-Wall', '-o', os.path.join(CALIB_LIB, 'libdeep_ep_calib.so'),
         os.path.join(CSRC, 'ep_calib.cpp')])
    run(['gcc', *C_CLIENT_FLAGS, '-o', os.path.join(LIB, 'abi_client'), os.path.join(CSRC, 'abi_client.c'),
         f'-L{LIB}', '-ldeep_ep_hip', f'-L{ROCM}/lib', '-lamdhip64', '-Wl,-rpath,$ORIGIN', f'-Wl,-rpath,{ROCM}/lib'])


if __name__ == '__main__':
    build()
    sys.exit(0)
