"""ctypes binding of libs2cnn_hip.so (the C ABI declared in include/s2cnn_hip.h).

There is no CPU fallback: if the library is not built, or a tensor is not a
float32 tensor on a GPU, the call raises.  Takes the place of the run-time
kernel compiler of the reference (s2cnn/utils/cuda.py:19-27).
"""
import ctypes
import os
from functools import lru_cache

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libs2cnn_hip.so")

_c_float_p = ctypes.c_void_p
_int, _long, _size_t, _vp = ctypes.c_int, ctypes.c_long, ctypes.c_size_t, ctypes.c_void_p

_MM_SIG = [_c_float_p, _c_float_p, _c_float_p, _int, _int, _int, _int, _vp]
_FT_SIG = [_c_float_p, _c_float_p, _c_float_p, _vp, _size_t, _int, _int, _long, _int, _vp]
_FT3_SIG = [_c_float_p, _c_float_p, _c_float_p, _c_float_p, _vp, _size_t, _int, _int, _long, _int, _vp]
_FT3R_SIG = [_c_float_p, _c_float_p, _c_float_p, _c_float_p, _vp, _size_t, _int, _int, _long, _vp]
_WS_SIG = [_int, _int, _long, _int]

SIGNATURES = {
    "s2cnn_abi_version": (_int, []),
    "s2cnn_strerror": (ctypes.c_char_p, [_int]),
    "s2cnn_so3_mm_fwd": (_int, _MM_SIG),
    "s2cnn_so3_mm_gradx": (_int, _MM_SIG),
    "s2cnn_so3_mm_grady": (_int, _MM_SIG),
    "s2cnn_so3_mm_real_fwd": (_int, _MM_SIG),
    "s2cnn_so3_mm_real_gradx": (_int, _MM_SIG),
    "s2cnn_so3_mm_real_grady": (_int, _MM_SIG),
    "s2cnn_so3_spectrum_to_real": (_int, [_c_float_p, _c_float_p, _int, _long, _vp]),
    "s2cnn_so3_spectrum_to_complex": (_int, [_c_float_p, _c_float_p, _int, _long, _vp]),
    "s2cnn_so3_rft_expand_real": (_int, [_c_float_p, _c_float_p, _c_float_p, _int, _int, _long, _vp]),
    "s2cnn_so3_rft_expand": (_int, [_c_float_p, _c_float_p, _c_float_p, _int, _int, _long, _vp]),
    "s2cnn_so3_rft_expand_real_grad": (_int, [_c_float_p, _c_float_p, _c_float_p, _int, _int, _long, _vp]),
    "s2cnn_s2_mm_fwd": (_int, _MM_SIG),
    "s2cnn_s2_mm_gradx": (_int, _MM_SIG),
    "s2cnn_s2_mm_grady": (_int, _MM_SIG),
    "s2cnn_s2_mm_real_fwd": (_int, _MM_SIG),
    "s2cnn_s2_mm_real_gradx": (_int, _MM_SIG),
    "s2cnn_s2_mm_real_grady": (_int, _MM_SIG),
    "s2cnn_so3_analysis_workspace": (_size_t, _WS_SIG),
    "s2cnn_so3_analysis": (_int, _FT3_SIG),
    "s2cnn_so3_analysis_static": (_int, [_c_float_p, _c_float_p, _c_float_p, _c_float_p, _int, _int, _long, _int, _vp]),
    "s2cnn_so3_synthesis_workspace": (_size_t, _WS_SIG),
    "s2cnn_so3_synthesis": (_int, _FT3_SIG),
    "s2cnn_so3_synthesis_real_bias": (_int, _FT3R_SIG[:-1] + [_c_float_p, _int, _vp]),
    "s2cnn_so3_synthesis_real_relu": (_int, _FT3R_SIG[:-1] + [_c_float_p, _int, _int, _vp]),
    "s2cnn_so3_analysis_real_masked": (_int, [_c_float_p] + _FT3R_SIG[:-1] + [_int, _vp]),
    "s2cnn_so3_relu_bits_bytes": (_size_t, [_int, _long]),
    "s2cnn_so3_synthesis_real_relu_bits": (_int, _FT3R_SIG[:4] + [_vp] + _FT3R_SIG[4:-1] + [_c_float_p, _int, _int, _vp]),
    "s2cnn_so3_analysis_real_masked_bits": (_int, [_c_float_p, _vp] + _FT3R_SIG[1:-1] + [_int, _vp]),
    "s2cnn_so3_analysis_prologue_available": (_int, [_int, _int]),
    "s2cnn_so3_integrate_affine_relu": (_int, [_c_float_p, _c_float_p, _int, _c_float_p, _c_float_p, _int, _long, _vp]),
    "s2cnn_volume_moments": (_int, [_c_float_p, _c_float_p, _long, _long, _vp]),
    "s2cnn_bn_forward_from_moments": (_int, [_c_float_p, _int, _int, _int, ctypes.c_double, _c_float_p, _c_float_p, _c_float_p, _c_float_p,
                                             ctypes.c_double, ctypes.c_double, _int, _c_float_p, _c_float_p, _vp]),
    "s2cnn_bn_backward_from_moments": (_int, [_c_float_p, _int, _int, _int, ctypes.c_double, _c_float_p, _c_float_p, _int, _c_float_p, _c_float_p, _vp]),
    "s2cnn_so3_synthesis_moment_parts": (_int, [_int, _int]),
    "s2cnn_so3_synthesis_real_moments": (_int, _FT3R_SIG[:-1] + [_c_float_p, _int, _c_float_p, _c_float_p, _c_float_p, _vp]),
    "s2cnn_so3_synthesis_real_basis_moment_parts": (_int, [_int, _int, _int]),
    "s2cnn_so3_synthesis_real_basis_moments": (_int, _FT3R_SIG[:-1] + [_c_float_p, _int, _c_float_p, _c_float_p, _c_float_p, _vp]),
    "s2cnn_bn_relu_grad_moments": (_int, [_c_float_p, _c_float_p, _c_float_p, _int, _c_float_p, _long, _long, _vp]),
    "s2cnn_so3_analysis_real_affine_relu": (_int, [_c_float_p, _c_float_p, _int] + _FT3R_SIG[1:-1] + [_int, _vp]),
    "s2cnn_so3_analysis_real_bn_relu_grad": (_int, [_c_float_p, _c_float_p, _c_float_p, _int] + _FT3R_SIG[1:-1] + [_int, _vp]),
    "s2cnn_so3_real_basis_transform_available": (_int, [_int, _int, _int]),
    "s2cnn_so3_analysis_real_basis": (_int, _FT3R_SIG),
    "s2cnn_so3_synthesis_real_basis": (_int, _FT3R_SIG[:-1] + [_c_float_p, _int, _vp]),
    "s2cnn_so3_packed_table_bytes": (_size_t, [_int, _int, _int]),
    "s2cnn_so3_pack_table": (_int, [_c_float_p, _c_float_p, _int, _int, _int, _vp]),
    "s2cnn_s2_analysis_workspace": (_size_t, _WS_SIG),
    "s2cnn_s2_analysis": (_int, _FT_SIG),
    "s2cnn_s2_synthesis_workspace": (_size_t, _WS_SIG),
    "s2cnn_s2_synthesis": (_int, _FT_SIG),
    "s2cnn_so3_integrate": (_int, [_c_float_p, _c_float_p, _c_float_p, _int, _long, _vp]),
    "s2cnn_so3_integrate_grad": (_int, [_c_float_p, _c_float_p, _c_float_p, _int, _long, _vp]),
}


@lru_cache(maxsize=1)
def lib():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libs2cnn_hip.so is not built (%s); run `python -m s2cnn_amd.csrc.build`. "
            "There is no CPU fallback." % LIB_PATH)
    handle = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    return handle


PROBE_LIB_PATH = os.path.join(_HERE, "csrc", "libs2cnn_probe.so")


@lru_cache(maxsize=1)
def probe_lib():
    """The measurement library (include/s2cnn_hip_probe.h): kernels with parts compiled out, for `bench.py --floor` only.
    Built on request (`python -m s2cnn_amd.csrc.build --probes`); nothing in the package calls it."""
    if not os.path.exists(PROBE_LIB_PATH):
        raise RuntimeError("libs2cnn_probe.so is not built (%s); run `python -m s2cnn_amd.csrc.build --probes`" % PROBE_LIB_PATH)
    handle = ctypes.CDLL(PROBE_LIB_PATH)
    handle.s2cnn_so3_fft64_probe.restype = _int
    handle.s2cnn_so3_fft64_probe.argtypes = [_c_float_p, _c_float_p, _c_float_p, _vp, _size_t, _long, _int, _int, _vp]
    return handle


class KernelTimer:
    """Optional per-call device timing: while active, every C-ABI call made through `call` is
    bracketed by two events recorded on the stream the kernels are launched on (torch's current
    stream).  Read the durations with `summary()` after a synchronize."""
    active = None

    def __init__(self):
        self.records = []

    def __enter__(self):
        KernelTimer.active = self
        return self

    def __exit__(self, *exc):
        KernelTimer.active = None

    def summary(self):
        out = {}
        for name, e0, e1 in self.records:
            out.setdefault(name, []).append(e0.elapsed_time(e1))
        return out


def call(name, *args):
    """Invoke one entry point of the library and raise on a non-zero return code."""
    fn = getattr(lib(), name)
    timer = KernelTimer.active
    if timer is None:
        check(fn(*args))
        return
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    check(fn(*args))
    e1.record()
    timer.records.append((name, e0, e1))


def check(code):
    if code != 0:
        raise RuntimeError("libs2cnn_hip: %s (code %d)" % (lib().s2cnn_strerror(code).decode(), code))


def require_gpu_f32(*tensors):
    """Operands must be float32 tensors on the current GPU: kernels are launched on the current device's current
    stream (as the reference's are, s2cnn/soft/so3_fft.py:341), so an operand elsewhere would be read across devices."""
    for t in tensors:
        if not (t.is_cuda and t.dtype == torch.float32):
            raise RuntimeError(
                "s2cnn_amd runs float32 tensors on the GPU only (got %s on %s); there is no CPU path"
                % (t.dtype, t.device))
        if t.device.index != torch.cuda.current_device():
            raise RuntimeError("operand on %s but the current device is cuda:%d: call inside torch.cuda.device(%d)"
                               % (t.device, torch.cuda.current_device(), t.device.index))


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def workspace(nbytes, device):
    """Scratch from torch's caching allocator (stream-ordered, so reuse after the call is safe)."""
    return torch.empty(max(int(nbytes), 8), dtype=torch.uint8, device=device)
