"""ctypes binding of libeshkol_gpu_hip.so, the MI355X backend behind Eshkol's
GPU C ABI (include/eshkol/backend/gpu/gpu_memory.h).

The product is the shared library; this module only loads it and gives the
tests and the benchmark a thin way to call it. It names things as the reference
header does (reference inc/eshkol/backend/gpu/gpu_memory.h): EshkolGPUBuffer,
eshkol_gpu_alloc, eshkol_gpu_matmul_f64, eshkol_matmul_dispatch, ...

There is no fallback: if the library has not been built, load() raises.
"""
import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "lib", "libeshkol_gpu_hip.so")

# EshkolGPUBackend / EshkolMemoryType / EshkolSyncDirection (gpu_memory.h)
GPU_NONE, GPU_METAL, GPU_CUDA, GPU_VULKAN, GPU_HIP = 0, 1, 2, 3, 4
MEM_HOST, MEM_HOST_PINNED, MEM_DEVICE, MEM_UNIFIED = 0, 1, 2, 3
SYNC_NONE, SYNC_HOST_TO_DEVICE, SYNC_DEVICE_TO_HOST, SYNC_BIDIRECTIONAL = 0, 1, 2, 3
DTYPE_F64, DTYPE_F32, DTYPE_F16, DTYPE_BF16, DTYPE_I8 = 0, 1, 2, 3, 4

u64, i64, i32, u32 = C.c_uint64, C.c_int64, C.c_int32, C.c_uint32
vp, dp = C.c_void_p, C.POINTER(C.c_double)


class EshkolGPUBuffer(C.Structure):
    _fields_ = [("host_ptr", vp), ("device_ptr", vp), ("size_bytes", C.c_size_t),
                ("mem_type", C.c_int), ("backend", C.c_int), ("flags", u32),
                ("backend_data", vp)]


class HipIgemmArgs(C.Structure):
    _fields_ = [("a_planes", vp), ("b_planes", vp), ("a_plane_stride", u64), ("b_plane_stride", u64),
                ("ldk", u32), ("M", u32), ("N", u32), ("n_out", u32),
                ("pair_first", vp), ("pair_a", vp), ("pair_b", vp),
                ("mode", i32), ("max_pairs", i32), ("modulus", vp), ("out_i32", vp), ("out_i8", vp),
                ("layout", i32), ("ldn", u32), ("out_rows", u32)]


class HipOzakiCrtStages(C.Structure):
    _fields_ = [("a_planes", vp), ("b_planes", vp), ("w_planes", vp), ("mu", vp), ("nu", vp),
                ("rows_a_padded", u64), ("rows_b_padded", u64), ("ldk", u64),
                ("num_moduli", i32), ("E", i32), ("layout", i32), ("w_rows", u64), ("w_ld", u64)]


class HipOzakiFastStages(C.Structure):
    _fields_ = [("a_planes", vp), ("b_planes", vp), ("w_planes", vp), ("shift_a", vp), ("shift_b", vp),
                ("rows_a_padded", u64), ("rows_b_padded", u64), ("ldk", u64),
                ("num_moduli", i32), ("E", i32), ("cap", i32), ("moduli", i32 * 16),
                ("layout", i32), ("w_rows", u64), ("w_ld", u64)]


class HipOzakiInt8Stages(C.Structure):
    _fields_ = [("a_slices", vp), ("b_slices", vp), ("products", vp), ("rmax", vp), ("cmax", vp),
                ("rows_a_padded", u64), ("rows_b_padded", u64), ("ldk", u64),
                ("s", i32), ("nbuf", i32), ("layout", i32), ("g_rows", u64), ("g_ld", u64)]


BUF = C.POINTER(EshkolGPUBuffer)

# name -> (restype, argtypes); every symbol the two public headers and the testing header declare
SIGNATURES = {
    # gpu_memory.h
    "eshkol_gpu_init": (C.c_int, []),
    "eshkol_gpu_shutdown": (None, []),
    "eshkol_gpu_get_backend": (C.c_int, []),
    "eshkol_gpu_backend_name": (C.c_char_p, [C.c_int]),
    "eshkol_gpu_backend_available": (C.c_int, [C.c_int]),
    "eshkol_gpu_supports_f64": (C.c_int, []),
    "eshkol_gpu_has_fp64": (C.c_int, []),
    "eshkol_gpu_alloc": (C.c_int, [C.c_size_t, C.c_int, BUF]),
    "eshkol_gpu_alloc_aligned": (C.c_int, [C.c_size_t, C.c_size_t, C.c_int, BUF]),
    "eshkol_gpu_free": (None, [BUF]),
    "eshkol_gpu_wrap_host": (C.c_int, [vp, C.c_size_t, BUF]),
    "eshkol_gpu_sync": (C.c_int, [BUF, C.c_int]),
    "eshkol_gpu_sync_async": (C.c_int, [BUF, C.c_int, vp]),
    "eshkol_gpu_wait": (None, [BUF]),
    "eshkol_gpu_matmul_f64": (C.c_int, [BUF, BUF, BUF, u64, u64, u64]),
    "eshkol_gpu_matmul_f32": (C.c_int, [BUF, BUF, BUF, u64, u64, u64]),
    "eshkol_gpu_matmul_backward_f64": (C.c_int, [BUF, BUF, BUF, BUF, BUF, u64, u64, u64]),
    "eshkol_gpu_resident_pin": (C.c_int, [vp, C.c_size_t]),
    "eshkol_gpu_resident_refresh": (C.c_int, [vp]),
    "eshkol_gpu_resident_unpin": (None, [vp]),
    "eshkol_gpu_resident_bytes": (C.c_size_t, []),
    "eshkol_gpu_set_threshold": (None, [C.c_size_t]),
    "eshkol_gpu_get_threshold": (C.c_size_t, []),
    "eshkol_gpu_should_use": (C.c_int, [C.c_size_t]),
    "eshkol_gpu_elementwise_f64": (C.c_int, [BUF, BUF, BUF, u64, C.c_int]),
    "eshkol_gpu_reduce_f64": (C.c_int, [BUF, BUF, u64, C.c_int]),
    "eshkol_gpu_reduce_axis_f64": (C.c_int, [BUF, BUF, u64, C.POINTER(u64), u64, C.c_int]),
    "eshkol_gpu_transpose_f64": (C.c_int, [BUF, BUF, u64, u64]),
    "eshkol_gpu_softmax_f64": (C.c_int, [BUF, BUF, u64, u64]),
    "eshkol_gpu_normalize_f64": (C.c_int, [BUF, BUF, u64, u64, C.c_double, C.c_double, C.c_double]),
    "eshkol_gpu_conv2d_backward_input_f64": (C.c_int, [BUF] * 3 + [u64] * 11),
    "eshkol_gpu_conv2d_backward_kernel_f64": (C.c_int, [BUF] * 3 + [u64] * 11),
    "eshkol_gpu_batchnorm_backward_f64": (C.c_int, [BUF] * 8 + [u64] * 2),
    "eshkol_gpu_layernorm_backward_f64": (C.c_int, [BUF] * 6 + [u64] * 2),
    "eshkol_matmul_dispatch": (None, [vp, vp, vp, u64, u64, u64, i32]),
    "eshkol_batch_matmul_dispatch": (None, [vp, vp, vp, i64, i64, i64, i64, i32]),
    # gpu_hip_tiers.h
    "eshkol_hip_get_stream": (vp, []),
    "hip_dgemm_f64": (C.c_int, [vp, vp, vp, u64, u64, u64, vp]),
    "hip_dgemm_f64_ex": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, vp]),
    "hip_dgemm_f64_batched": (C.c_int, [vp, vp, vp, u64, u64, u64, u64, vp]),
    "hip_dgemm_set_fast_path": (None, [C.c_int]),
    "hip_sgemm_f32": (C.c_int, [vp, vp, vp, u64, u64, u64, vp]),
    "hip_transpose_f64": (C.c_int, [vp, vp, u64, u64, vp]),
    "hip_colabsmax_f64": (C.c_int, [vp, u64, u64, C.c_double, vp, vp]),
    "hip_ozaki_crt_split_kmajor_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, vp]),
    "hip_ozaki_slice_kmajor_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, vp]),
    "hip_convert_f64_to_16_kmajor": (C.c_int, [vp, vp, u64, u64, u64, u64, C.c_int, vp]),
    "hip_rowabsmax_f64": (C.c_int, [vp, u64, u64, C.c_double, vp, vp]),
    "hip_elementwise_f64": (C.c_int, [vp, vp, vp, u64, C.c_int, vp]),
    "hip_bias_act_f64": (C.c_int, [vp, vp, u64, u64, C.c_int, vp]),
    "hip_igemm_i8": (C.c_int, [C.POINTER(HipIgemmArgs), vp]),
    "hip_ozaki_crt_split_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, vp]),
    "hip_ozaki_crt_reconstruct_f64": (C.c_int, [vp, u64, u64, C.c_int, dp, dp, C.c_double, C.c_double,
                                                C.c_double, vp, vp, vp, C.c_int, vp, vp]),
    "hip_matmul_ozaki_crt_f64": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, vp, C.c_int, vp]),
    "hip_ozaki_crt_last_stages": (C.c_int, [C.POINTER(HipOzakiCrtStages)]),
    "hip_matmul_ozaki_fast_f64": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, vp]),
    "hip_matmul_ozaki_fast_f64_ex": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, C.c_int, vp]),
    "hip_ozaki_fast_last_stages": (C.c_int, [C.POINTER(HipOzakiFastStages)]),
    "hip_ozaki_crt_set_aligned_weights": (C.c_int, [C.c_int]),
    "hip_select_tier_for_budget": (C.c_int, [u64, u64, u64, C.c_double, C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                             C.POINTER(C.c_double)]),
    "hip_ozaki_fast_plan": (C.c_int, [u64, C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "hip_ozaki_slice_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, vp]),
    "hip_ozaki_reconstruct_f64": (C.c_int, [vp, vp, vp, C.c_int, vp, vp, u64, u64, vp]),
    "hip_matmul_ozaki_int8_f64": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, vp]),
    "hip_ozaki_int8_last_stages": (C.c_int, [C.POINTER(HipOzakiInt8Stages)]),
    "hip_matmul_reduced_f64": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, vp]),
    "hip_matmul_reduced_f64_noalloc": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, vp]),
    "hip_matmul_reduced_f64_noalloc_limit": (C.c_size_t, []),
    "hip_matmul_ozaki_crt_f64_ex": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, C.c_int, C.c_int,
                                              vp, C.c_int, vp]),
    "hip_matmul_ozaki_int8_f64_ex": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, C.c_int, vp]),
    "hip_matmul_reduced_f64_ex": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, C.c_int, C.c_int, vp]),
    "hip_matmul_backward_f64": (C.c_int, [vp, vp, vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, vp]),
    "hip_hgemm_16": (C.c_int, [vp, vp, u64, u64, u64, u64, C.c_int, vp, vp]),
    "hip_convert_f64_to_16": (C.c_int, [vp, vp, u64, u64, u64, u64, C.c_int, vp]),
    "hip_igemm_set_persistent": (None, [C.c_int]),
    "hip_ozaki_crt_prepare_operand_b": (C.c_int, [vp, u64, u64, C.c_int, C.c_int, u64, C.POINTER(vp), vp]),
    "hip_matmul_ozaki_crt_prepared_f64": (C.c_int, [vp, vp, vp, u64, u64, u64, C.c_int, C.c_int, C.c_int, vp, C.c_int, vp]),
    "hip_ozaki_crt_release_prepared": (None, [vp]),
    "hip_ozaki_fast_split_planes_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, C.c_int, C.c_int, vp]),
    "hip_ozaki_fast_reconstruct_f64": (C.c_int, [vp, u64, u64, u64, C.c_int, vp, vp, vp, vp]),
    "hip_igemm_set_direct": (None, [C.c_int]),
    "hip_igemm_set_cu_limit": (None, [C.c_int]),
    "hip_hgemm_set_direct": (None, [C.c_int]),
    "hip_reduced_set_thin": (None, [C.c_int]),
    "hip_hgemm_plane_layout": (C.c_int, [u64, u64, u64]),
    "hip_hgemm_16_batched": (C.c_int, [vp, vp, u64, u64, u64, u64, u64, u64, u64, C.c_int, C.c_int, vp, vp]),
    "hip_convert_f64_to_16_planes": (C.c_int, [vp, vp, u64, u64, u64, u64, u64, C.c_int, C.c_int, C.c_int, vp]),
    "hip_matmul_reduced_f64_batched": (C.c_int, [vp, vp, vp, u64, u64, u64, u64, C.c_int, C.c_int, vp]),
    "hip_igemm_plane_layout": (C.c_int, [u64, u64, C.c_int]),
    "hip_igemm_plane_layout_single": (C.c_int, [u64, u64, u64, C.c_int]),
    "hip_ozaki_crt_split_planes_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, C.c_int, C.c_int, vp]),
    "hip_ozaki_slice_planes_f64": (C.c_int, [vp, u64, u64, vp, C.c_int, vp, u64, u64, C.c_int, C.c_int, vp]),
    "hip_dgemm_set_tail_split": (None, [C.c_int]),
    "hip_dgemm_set_small_tile": (None, [C.c_int]),
    "hip_dgemm_set_prefetch_depth": (None, [C.c_int]),
    "hip_dgemm_set_thin_rows": (None, [C.c_int]),
    "hip_dgemm_set_thin_rows_klast": (None, [C.c_int]),
    "hip_dgemm_set_thin_chunks": (None, [C.c_int]),
    "hip_igemm_set_thin_variant": (None, [C.c_int]),
    "hip_ozaki_crt_set_host_pass": (None, [C.c_int]),
    "hip_ozaki_crt_set_fused_scan": (None, [C.c_int]),
    "hip_igemm_set_prefetch": (None, [C.c_int]),
}

_lib = None
_hip = None


def load():
    """Load the shared library (RTLD_GLOBAL, so a host runtime loaded earlier can
    satisfy eshkol_matmul_f64) and attach the C signatures. Raises if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libeshkol_gpu_hip.so is not built (%s); run `python -m eshkol_amd.build`. "
            "There is no CPU fallback in this package." % LIB_PATH)
    lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def load_probe():
    """The device probe of the benchmark (libeshkol_gpu_probe.so: register-only MFMA
    loops and a large copy). Not part of the product library."""
    path = os.path.join(PKG, "lib", "libeshkol_gpu_probe.so")
    if not os.path.exists(path):
        raise RuntimeError("libeshkol_gpu_probe.so is not built (%s); run `python -m eshkol_amd.build`" % path)
    probe = C.CDLL(path)
    probe.hip_probe_peak.restype = C.c_int
    probe.hip_probe_peak.argtypes = [C.c_int, C.c_int, dp, vp]
    probe.hip_probe_coissue.restype = C.c_int
    probe.hip_probe_coissue.argtypes = [C.c_int, C.c_int, C.c_int, dp, dp, dp, vp]
    return probe


def hip_runtime():
    """The HIP runtime the library itself is linked against, for memcpy/events."""
    global _hip
    if _hip is not None:
        return _hip
    h = C.CDLL("libamdhip64.so", mode=C.RTLD_GLOBAL)
    h.hipMemcpy.argtypes = [vp, vp, C.c_size_t, C.c_int]
    h.hipMemcpy.restype = C.c_int
    h.hipMemset.argtypes = [vp, C.c_int, C.c_size_t]
    h.hipDeviceSynchronize.restype = C.c_int
    h.hipStreamSynchronize.argtypes = [vp]
    h.hipStreamCreate.argtypes = [C.POINTER(vp)]
    h.hipStreamDestroy.argtypes = [vp]
    h.hipEventCreate.argtypes = [C.POINTER(vp)]
    h.hipEventRecord.argtypes = [vp, vp]
    h.hipEventSynchronize.argtypes = [vp]
    h.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), vp, vp]
    h.hipEventDestroy.argtypes = [vp]
    h.hipGetDeviceCount.argtypes = [C.POINTER(C.c_int)]
    _hip = h
    return h


H2D, D2H, D2D = 1, 2, 3


def init():
    """eshkol_gpu_init(); raises unless the HIP backend came up."""
    lib = load()
    if lib.eshkol_gpu_init() != 1 or lib.eshkol_gpu_get_backend() != GPU_HIP:
        raise RuntimeError("eshkol_gpu_init(): no gfx950 device; the HIP backend is not active")
    return lib


class DeviceArray:
    """A device buffer obtained through eshkol_gpu_alloc(ESHKOL_MEM_DEVICE)."""

    def __init__(self, shape, dtype=np.float64):
        self.lib = load()
        self.shape = tuple(int(s) for s in (shape if hasattr(shape, "__len__") else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        self.buf = EshkolGPUBuffer()
        if self.lib.eshkol_gpu_alloc(max(self.nbytes, 1), MEM_DEVICE, C.byref(self.buf)) != 0:
            raise MemoryError("eshkol_gpu_alloc(%d bytes) failed" % self.nbytes)

    @property
    def ptr(self):
        return self.buf.device_ptr

    @classmethod
    def from_host(cls, arr):
        arr = np.ascontiguousarray(arr)
        d = cls(arr.shape, arr.dtype)
        d.upload(arr)
        return d

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        assert arr.nbytes == self.nbytes
        rc = hip_runtime().hipMemcpy(self.ptr, arr.ctypes.data, self.nbytes, H2D)
        if rc != 0:
            raise RuntimeError("hipMemcpy H2D failed: %d" % rc)

    def download(self):
        out = np.empty(self.shape, self.dtype)
        rc = hip_runtime().hipMemcpy(out.ctypes.data, self.ptr, self.nbytes, D2H)
        if rc != 0:
            raise RuntimeError("hipMemcpy D2H failed: %d" % rc)
        return out

    def free(self):
        if self.buf.device_ptr:
            self.lib.eshkol_gpu_free(C.byref(self.buf))

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def download_raw(ptr, shape, dtype):
    """Copy device memory the library owns (stage outputs) to a new host array."""
    out = np.empty(shape, dtype)
    rc = hip_runtime().hipMemcpy(out.ctypes.data, ptr, out.nbytes, D2H)
    if rc != 0:
        raise RuntimeError("hipMemcpy D2H failed: %d" % rc)
    return out


def deinterleave(planes, layout):
    """Operand planes [n][rows][ldk] as the library stores them -> plain [n][rows][ldk].
    layout 1 (HipIgemmArgs.layout): rows in blocks of 32, inside a block the 16-byte
    k-chunks slow and the row fast."""
    if not layout:
        return planes
    n, rows, ldk = planes.shape
    item = planes.dtype.itemsize
    per = 16 // item                                  # elements per 16-byte chunk
    y = planes.reshape(n, rows // 32, ldk // per, 32, per).transpose(0, 1, 3, 2, 4)
    return np.ascontiguousarray(y).reshape(n, rows, ldk)


def synchronize():
    hip_runtime().hipDeviceSynchronize()


def matmul_dispatch(A, B, dtype=DTYPE_F64):
    """eshkol_matmul_dispatch on host arrays: returns C = A @ B as float64."""
    lib = load()
    A = np.ascontiguousarray(A, dtype=np.float64)
    B = np.ascontiguousarray(B, dtype=np.float64)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    Cc = np.empty((M, N), dtype=np.float64)
    lib.eshkol_matmul_dispatch(A.ctypes.data, B.ctypes.data, Cc.ctypes.data, M, K, N, dtype)
    return Cc


class Timer:
    """HIP events recorded on the library's stream."""

    def __init__(self):
        self.h = hip_runtime()
        self.stream = load().eshkol_hip_get_stream()
        self.e0, self.e1 = vp(), vp()
        self.h.hipEventCreate(C.byref(self.e0))
        self.h.hipEventCreate(C.byref(self.e1))

    def start(self):
        self.h.hipEventRecord(self.e0, self.stream)

    def stop(self):
        self.h.hipEventRecord(self.e1, self.stream)
        self.h.hipEventSynchronize(self.e1)
        ms = C.c_float()
        self.h.hipEventElapsedTime(C.byref(ms), self.e0, self.e1)
        return float(ms.value)
