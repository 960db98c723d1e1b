"""cactus_amd -- MI355X (gfx950) backend for Cactus's quantized MUL_MAT path.

The product is two shared libraries built from cactus_amd/csrc:

  lib/libcactus_hip.so   hand-written HIP kernels behind the C-ABI of include/cactus_hip.h
  lib/libggml-hip.so     the ggml backend (reg / device / buffer type / graph_compute) on top of it

This Python package is a thin ctypes binding of the C-ABI for tests and benchmarks.  There is no CPU or
PyTorch fallback: if the library is missing or no gfx950 device is present, loading raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(HERE, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libcactus_hip.so")
BACKEND_LIB = os.path.join(LIB_DIR, "libggml-hip.so")

F32, Q4_0, Q8_0, Q4_K, Q6_K, Q8_K = 0, 2, 8, 12, 14, 15
Q5_0, Q5_K, IQ4_NL = 6, 13, 20
Q2_K, Q3_K, IQ4_XS = 10, 11, 23
Q6_K_PLANES = 114           # CHIP_TYPE_Q6_K_PLANES: Q6_K rows repacked by chip_repack_q6_K (no type of the reference)
Q4_1, Q5_1, Q8_1 = 3, 7, 9
F16 = 1
CHIP_OK, CHIP_EINVAL, CHIP_EUNSUPPORTED, CHIP_ENOMEM = 0, -1, -2, -3        # include/cactus_hip.h
TYPE_NAMES = {F32: "f32", Q4_0: "q4_0", Q8_0: "q8_0", Q4_K: "q4_K", Q6_K: "q6_K", Q8_K: "q8_K",
              Q5_0: "q5_0", Q5_K: "q5_K", IQ4_NL: "iq4_nl", Q4_1: "q4_1", Q5_1: "q5_1", Q8_1: "q8_1", F16: "f16", Q3_K: "q3_K",
              Q2_K: "q2_K", IQ4_XS: "iq4_xs", Q6_K_PLANES: "q6_K_planes"}
WEIGHT_TYPES = (Q4_0, Q8_0, Q4_K, Q6_K, Q5_0, Q5_K, IQ4_NL, Q4_1, Q5_1, Q3_K, Q2_K, IQ4_XS, F16)

# every symbol include/cactus_hip.h declares
EXPORTS = (
    "chip_init", "chip_device_count", "chip_get_device_info", "chip_error_string", "chip_malloc", "chip_free",
    "chip_memcpy_h2d", "chip_memcpy_d2h", "chip_memcpy_d2d", "chip_memset", "chip_stream_create",
    "chip_stream_destroy", "chip_stream_synchronize", "chip_host_malloc", "chip_host_free", "chip_event_create",
    "chip_event_destroy", "chip_event_record", "chip_event_synchronize", "chip_stream_wait_event", "chip_block_elems", "chip_block_bytes", "chip_row_size",
    "chip_vec_dot_type", "chip_mul_mat_supported", "chip_quantize_q8_0", "chip_quantize_q8_K",
    "chip_quantize_q8_1", "chip_convert_f32_to_f16",
    "chip_mul_mat_workspace_size", "chip_mul_mat_workspace_size_n", "chip_mul_mat", "chip_mul_mat_prepare", "chip_mul_mat_run", "chip_mul_mat_run_ws", "chip_mul_mat_pair", "chip_mul_mat_pair_silu_mul", "chip_mul_mat_pair_silu_mul_supported", "chip_mul_mat_store_t", "chip_mul_mat_group", "chip_mul_mat_group_rope", "chip_mul_mat_group_rope_norm", "chip_mul_mat_pair_silu_mul_norm", "chip_norm_before_supported", "chip_mul_mat_add", "chip_mul_mat_add_supported", "chip_mul_mat_group_run", "chip_mul_mat_noalloc", "chip_mul_mat_noalloc_max_workspace", "chip_mul_mat_id",
    "chip_mul_mat_id_workspace_size", "chip_rms_norm", "chip_add", "chip_mul", "chip_silu", "chip_rms_norm_mul", "chip_silu_mul", "chip_add_rms_norm_mul", "chip_rms_norm_quantized", "chip_silu_mul_quantized", "chip_scale", "chip_gelu_table", "chip_gelu",
    "chip_soft_max", "chip_cpy", "chip_rope", "chip_rope_table", "chip_rope_apply", "chip_rope_apply_store", "chip_rope_apply_two", "chip_get_rows", "chip_mul_mat_f16_batched", "chip_mul_mat_f16_batched_workspace_size", "chip_mul_mat_f16_batched_two_copies", "chip_mul_mat_f16_batched_second_copy_supported",
    "chip_repack_q6_K", "chip_block_isums", "chip_verify_force_q6k_matrix_core",
    "chip_workspace_to_blocks",
)


class DeviceInfo(C.Structure):
    _fields_ = [("device", C.c_int), ("compute_units", C.c_int), ("wavefront_size", C.c_int),
                ("max_lds_per_block", C.c_int), ("clock_khz", C.c_int), ("xcd_count", C.c_int),
                ("hbm_total", C.c_size_t), ("hbm_free", C.c_size_t), ("name", C.c_char * 128), ("arch", C.c_char * 64)]


class Mat(C.Structure):
    """struct chip_mat: one member of chip_mul_mat_group."""
    _fields_ = [("type", C.c_int), ("W", C.c_void_p), ("nb01", C.c_size_t), ("N", C.c_int64), ("y", C.c_void_p),
                ("ldy", C.c_int64), ("y_f16_t", C.c_void_p), ("ld16", C.c_int64)]


class RopeOperand(C.Structure):
    """struct chip_rope_operand: one of the two tensors of chip_rope_apply_two."""
    _fields_ = [("x", C.c_void_p), ("ldx1", C.c_int64), ("ldx2", C.c_int64), ("ne1", C.c_int64), ("y", C.c_void_p),
                ("ldy1", C.c_int64), ("ldy2", C.c_int64), ("y_f16", C.c_void_p), ("ld16_1", C.c_int64), ("ld16_2", C.c_int64)]


class RopeAfter(C.Structure):
    """struct chip_rope_after: the ROPE node behind a member of chip_mul_mat_group_rope."""
    _fields_ = [("table", C.c_void_p), ("head_dim", C.c_int64), ("n_dims", C.c_int), ("mode", C.c_int), ("y", C.c_void_p),
                ("ldy", C.c_int64), ("y_f16", C.c_void_p), ("ld16", C.c_int64)]


class NormBefore(C.Structure):
    """struct chip_norm_before: the RMS norm and weight MUL run in a projection's prologue."""
    _fields_ = [("w", C.c_void_p), ("eps", C.c_float), ("y", C.c_void_p), ("ldy", C.c_int64)]


class ChipError(RuntimeError):
    pass


def build():
    """Compile the libraries in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
    import subprocess
    subprocess.check_call(["make", "-C", os.path.join(HERE, "csrc"), "-j8", "all"])


def load_library(path=KERNEL_LIB):
    """dlopen libcactus_hip.so and declare the prototypes.  Raises if the library has not been built."""
    if not os.path.exists(path):
        raise ChipError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                        "(there is no fallback implementation)" % path)
    L = C.CDLL(path)
    vp, i64, sz, i32 = C.c_void_p, C.c_int64, C.c_size_t, C.c_int
    L.chip_init.argtypes = [i32]
    L.chip_get_device_info.argtypes = [C.POINTER(DeviceInfo)]
    L.chip_error_string.restype = C.c_char_p
    L.chip_error_string.argtypes = [i32]
    L.chip_malloc.argtypes = [C.POINTER(vp), sz]
    L.chip_free.argtypes = [vp]
    for n in ("chip_memcpy_h2d", "chip_memcpy_d2h", "chip_memcpy_d2d"):
        getattr(L, n).argtypes = [vp, vp, sz, vp]
    L.chip_memset.argtypes = [vp, i32, sz, vp]
    L.chip_stream_create.argtypes = [C.POINTER(vp)]
    L.chip_stream_destroy.argtypes = [vp]
    L.chip_stream_synchronize.argtypes = [vp]
    L.chip_host_malloc.argtypes = [C.POINTER(vp), sz]
    L.chip_host_free.argtypes = [vp]
    L.chip_event_create.argtypes = [C.POINTER(vp)]
    L.chip_event_destroy.argtypes = [vp]
    L.chip_event_record.argtypes = [vp, vp]
    L.chip_event_synchronize.argtypes = [vp]
    L.chip_stream_wait_event.argtypes = [vp, vp]
    L.chip_block_elems.argtypes = [i32]
    L.chip_block_bytes.restype = sz
    L.chip_block_bytes.argtypes = [i32]
    L.chip_row_size.restype = sz
    L.chip_row_size.argtypes = [i32, i64]
    L.chip_vec_dot_type.argtypes = [i32]
    L.chip_mul_mat_supported.argtypes = [i32, i64]
    L.chip_quantize_q8_0.argtypes = [vp, i64, i64, i64, vp, vp]
    L.chip_quantize_q8_K.argtypes = [vp, i64, i64, i64, vp, vp]
    L.chip_quantize_q8_1.argtypes = [vp, i64, i64, i64, vp, vp]
    L.chip_convert_f32_to_f16.argtypes = [vp, i64, i64, i64, vp, vp]
    L.chip_mul_mat_workspace_size.restype = sz
    L.chip_mul_mat_workspace_size.argtypes = [i32, i64, i64]
    L.chip_mul_mat_workspace_size_n.restype = sz
    L.chip_mul_mat_workspace_size_n.argtypes = [i32, i64, i64, i64]
    L.chip_mul_mat.argtypes = [i32, vp, sz, i64, i64, vp, i64, i64, vp, i64, vp, sz, vp]
    L.chip_mul_mat_group.argtypes = [C.POINTER(Mat), i32, i64, vp, i64, i64, vp, sz, vp]
    L.chip_mul_mat_group_run.argtypes = [C.POINTER(Mat), i32, i64, i64, vp, sz, vp]
    L.chip_mul_mat_noalloc.argtypes = [i32, vp, sz, i64, i64, vp, i64, i64, vp, i64, vp]
    L.chip_mul_mat_noalloc_max_workspace.restype = sz
    L.chip_mul_mat_noalloc_max_workspace.argtypes = []
    L.chip_mul_mat_prepare.argtypes = [i32, i64, vp, i64, i64, vp, sz, vp]
    L.chip_mul_mat_run.argtypes = [i32, vp, sz, i64, i64, i64, vp, vp, i64, vp]
    L.chip_mul_mat_run_ws.argtypes = [i32, vp, sz, i64, i64, i64, vp, sz, vp, i64, vp]
    L.chip_mul_mat_group_rope.argtypes = [C.POINTER(Mat), C.POINTER(RopeAfter), i32, i64, vp, i64, i64, vp, sz, vp]
    L.chip_mul_mat_pair.argtypes = [i32, vp, vp, sz, i64, i64, vp, i64, i64, vp, vp, i64, vp, sz, vp]
    L.chip_mul_mat_pair_silu_mul.argtypes = [i32, vp, vp, sz, i64, i64, vp, i64, i64, vp, i64, vp, sz, vp]
    L.chip_mul_mat_pair_silu_mul_supported.argtypes = [i32, i64, i64, i64]
    L.chip_mul_mat_group_rope_norm.argtypes = [C.POINTER(Mat), C.POINTER(RopeAfter), C.POINTER(NormBefore), i32, i64, vp, i64, i64, vp, sz, vp]
    L.chip_mul_mat_pair_silu_mul_norm.argtypes = [i32, vp, vp, sz, i64, i64, vp, i64, i64, C.POINTER(NormBefore), vp, i64, vp, sz, vp]
    L.chip_norm_before_supported.argtypes = [i32, i64, i64]
    L.chip_mul_mat_add_supported.argtypes = [i32, i64, i64, i64]
    L.chip_mul_mat_add.argtypes = [i32, vp, sz, i64, i64, vp, i64, i64, vp, i64, vp, i64, vp, sz, vp]
    L.chip_mul_mat_store_t.argtypes = [i32, vp, sz, i64, i64, vp, i64, i64, vp, i64, vp, i64, vp, sz, vp]
    L.chip_rms_norm.argtypes = [vp, i64, i64, i64, C.c_float, vp, i64, vp]
    L.chip_add.argtypes = [vp, i64, vp, i64, i64, i64, i64, vp, i64, vp]
    L.chip_mul.argtypes = [vp, i64, vp, i64, i64, i64, i64, vp, i64, vp]
    L.chip_silu.argtypes = [vp, i64, i64, i64, vp, i64, vp]
    L.chip_rms_norm_mul.argtypes = [vp, i64, i64, i64, C.c_float, vp, vp, i64, vp, i64, vp]
    L.chip_silu_mul.argtypes = [vp, i64, vp, i64, i64, i64, vp, i64, vp]
    L.chip_add_rms_norm_mul.argtypes = [vp, i64, vp, i64, vp, i64, i64, i64, C.c_float, vp, vp, i64, vp]
    L.chip_scale.argtypes = [vp, i64, i64, i64, C.c_float, vp, i64, vp]
    L.chip_rms_norm_quantized.argtypes = [vp, i64, vp, i64, vp, i64, i64, i64, C.c_float, vp, vp, i64, i32, vp, sz, vp]
    L.chip_silu_mul_quantized.argtypes = [vp, i64, vp, i64, i64, i64, vp, i64, i32, vp, sz, vp]
    L.chip_gelu_table.argtypes = [vp]
    L.chip_gelu.argtypes = [vp, i64, i64, i64, vp, vp, i64, vp]
    L.chip_soft_max.argtypes = [vp, i64, vp, i32, i64, i64, i64, C.c_float, C.c_float, vp, i64, vp]
    L.chip_cpy.argtypes = [vp, i32, C.POINTER(i64), C.POINTER(i64), vp, i32, C.POINTER(i64), C.POINTER(i64), vp]
    L.chip_rope.argtypes = [vp, i64, i64, vp, vp, i64, i64, i64, i32, i32, i32] + [C.c_float] * 6 + [vp, i64, i64, vp]
    L.chip_rope_table.argtypes = [vp, vp, i64, i32, i32] + [C.c_float] * 6 + [vp, vp]
    L.chip_rope_apply.argtypes = [vp, i64, i64, vp, i64, i64, i64, i32, i32, vp, i64, i64, vp]
    L.chip_rope_apply_store.argtypes = [vp, i64, i64, vp, i64, i64, i64, i32, i32, vp, i64, i64, vp, i64, i64, vp]
    L.chip_rope_apply_two.argtypes = [C.POINTER(RopeOperand), C.POINTER(RopeOperand), vp, i64, i64, i32, i32, vp]
    L.chip_get_rows.argtypes = [i32, vp, sz, sz, sz, i64, i64, vp, i64, i64, i64, i64, i64, vp, i64, i64, i64, vp]
    L.chip_mul_mat_f16_batched.argtypes = [vp, sz, sz, i64, i64, i64, vp, i64, i64, i64, i64, vp, i64, i64, vp, sz, vp]
    L.chip_mul_mat_f16_batched_workspace_size.restype = sz
    L.chip_mul_mat_f16_batched_second_copy_supported.argtypes = [i64, i64, i64]
    L.chip_mul_mat_f16_batched_two_copies.argtypes = [vp, sz, sz, i64, i64, i64, vp, i64, i64, i64, i64, vp, i64, i64, vp, i64, i64, vp, sz, vp]
    L.chip_mul_mat_f16_batched_workspace_size.argtypes = [i64, i64, i64, i64, i64]
    L.chip_mul_mat_id_workspace_size.restype = sz
    L.chip_mul_mat_id_workspace_size.argtypes = [i32, i64, i64, i64, i64, i64]
    L.chip_mul_mat_id.argtypes = [i32, vp, sz, sz, i64, i64, i64, vp, i64, i64, vp, i64, i64, i64, vp, i64, vp, sz, vp]
    L.chip_repack_q6_K.argtypes = [vp, sz, vp, sz, i64, i64, i32, vp]
    L.chip_block_isums.argtypes = [i32, vp, sz, i64, i64, vp, i64, vp, vp, vp]
    L.chip_verify_force_q6k_matrix_core.argtypes = [i32]
    L.chip_workspace_to_blocks.argtypes = [i32, i64, i64, vp, vp, vp]
    return L


class DeviceBuffer:
    """A hipMalloc'd region owned through the C-ABI."""

    def __init__(self, dev, nbytes):
        self.dev, self.nbytes = dev, int(nbytes)
        p = C.c_void_p()
        dev.check(dev.lib.chip_malloc(C.byref(p), max(self.nbytes, 16)))
        self.ptr = p.value

    def upload(self, arr, offset=0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= max(self.nbytes, 16)
        self.dev.check(self.dev.lib.chip_memcpy_h2d(self.ptr + offset, arr.ctypes.data, arr.nbytes, None))
        return self

    def download(self, dtype, count, offset=0):
        out = np.empty(count, dtype)
        assert offset + out.nbytes <= max(self.nbytes, 16)
        self.dev.check(self.dev.lib.chip_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes, None))
        return out

    def free(self):
        if self.ptr:
            self.dev.lib.chip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Device:
    """One gfx950 GPU seen through the C-ABI; numpy in, numpy out (host<->device copies are synchronous)."""

    def __init__(self, ordinal=0):
        self.lib = load_library()
        rc = self.lib.chip_init(ordinal)
        if rc != 0:
            raise ChipError("chip_init(%d) failed: %s" % (ordinal, self.error_string(rc)))
        self.info = DeviceInfo()
        self.check(self.lib.chip_get_device_info(C.byref(self.info)))

    def error_string(self, rc):
        return self.lib.chip_error_string(rc).decode()

    def check(self, rc):
        if rc != 0:
            raise ChipError("libcactus_hip: %s (code %d)" % (self.error_string(rc), rc))

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        return DeviceBuffer(self, arr.nbytes).upload(arr)

    def sync(self, stream=None):
        self.check(self.lib.chip_stream_synchronize(stream))

    def row_size(self, t, k):
        return self.lib.chip_row_size(t, k)

    # -- the hot path -------------------------------------------------------------------------------------
    def quantize(self, act_type, x):
        """x fp32 [n, K] -> uint8 [n, row_size] in the reference block layout."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        dx = self.to_device(x)
        rs = self.row_size(act_type, k)
        dy = self.alloc(n * rs)
        fn = {Q8_0: self.lib.chip_quantize_q8_0, Q8_K: self.lib.chip_quantize_q8_K,
              Q8_1: self.lib.chip_quantize_q8_1, F16: self.lib.chip_convert_f32_to_f16}[act_type]
        self.check(fn(dx.ptr, k, n, k, dy.ptr, None))
        self.sync()
        return dy.download(np.uint8, n * rs).reshape(n, rs)

    def mul_mat(self, wtype, W, x, dW=None, want_workspace_blocks=False, split_k=True):
        """LM_GGML_OP_MUL_MAT: W uint8 [N, row_size(wtype, K)] (or a DeviceBuffer via dW), x fp32 [n, K] -> y [n, N].
        split_k=False gives the library only the activation workspace, so a GEMM never splits K."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        if dW is None:
            W = np.ascontiguousarray(W, np.uint8)
            N = W.shape[0]
            dW = self.to_device(W)
        else:
            N = dW.nbytes // self.row_size(wtype, k)
        nb01 = self.row_size(wtype, k)
        dx = self.to_device(x)
        dy = self.alloc(n * N * 4)
        wsz = self.lib.chip_mul_mat_workspace_size_n(wtype, k, N, n) if split_k else self.lib.chip_mul_mat_workspace_size(wtype, k, n)
        ws = self.alloc(wsz)
        self.check(self.lib.chip_mul_mat(wtype, dW.ptr, nb01, k, N, dx.ptr, k, n, dy.ptr, N, ws.ptr, wsz, None))
        self.sync()
        y = dy.download(np.float32, n * N).reshape(n, N)
        if want_workspace_blocks:
            at = self.lib.chip_vec_dot_type(wtype)
            rs = self.row_size(at, k)
            db = self.alloc(n * rs)
            self.check(self.lib.chip_workspace_to_blocks(wtype, k, n, ws.ptr, db.ptr, None))
            self.sync()
            return y, db.download(np.uint8, n * rs).reshape(n, rs)
        return y

    # -- element-wise ops next to the matmuls ---------------------------------------------------------------
    def mul_mat_store_t(self, wtype, W, x, ld16):
        """chip_mul_mat_store_t: returns (y fp32 [n, N], the fp16 matrix [N, ld16] whose first n columns hold y transposed;
        the other columns keep the 0x7bff pattern they were filled with)."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        W = np.ascontiguousarray(W, np.uint8)
        N = W.shape[0]
        dW, dx, dy = self.to_device(W), self.to_device(x), self.alloc(n * N * 4)
        dh = self.to_device(np.full(N * ld16, 0x7bff, np.uint16))
        wsz = self.lib.chip_mul_mat_workspace_size_n(wtype, k, N, n)
        ws = self.alloc(wsz)
        self.check(self.lib.chip_mul_mat_store_t(wtype, dW.ptr, self.row_size(wtype, k), k, N, dx.ptr, k, n, dy.ptr, N, dh.ptr, ld16,
                                                 ws.ptr, wsz, None))
        self.sync()
        return dy.download(np.float32, n * N).reshape(n, N), dh.download(np.uint16, N * ld16).reshape(N, ld16)

    def mul_mat_group(self, members, x, ld16=0, prepared=False):
        """chip_mul_mat_group: members = [(wtype, W uint8 [N, row_size]), ...] on the activation rows x fp32 [n, K].
        Returns a list of y fp32 [n, N]; with ld16 > 0 the last member also stores its transposed fp16 copy and the list
        ends with that matrix [N, ld16] (untouched columns keep 0x7bff).  prepared: chip_mul_mat_prepare first, then
        chip_mul_mat_group_run over the workspace rows."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        dx = self.to_device(x)
        arr = (Mat * len(members))()
        keep, outs = [], []
        wsz = 0
        for i, (wt, W) in enumerate(members):
            W = np.ascontiguousarray(W, np.uint8)
            N = W.shape[0]
            dW, dy = self.to_device(W), self.alloc(n * N * 4)
            keep.append(dW)
            outs.append((dy, N))
            arr[i] = Mat(wt, dW.ptr, self.row_size(wt, k), N, dy.ptr, N, None, 0)
            wsz = max(wsz, self.lib.chip_mul_mat_workspace_size_n(wt, k, N, n))
        dh = None
        if ld16:
            dh = self.to_device(np.full(outs[-1][1] * ld16, 0x7bff, np.uint16))
            arr[len(members) - 1].y_f16_t = dh.ptr
            arr[len(members) - 1].ld16 = ld16
        ws = self.alloc(wsz)
        if prepared:
            self.check(self.lib.chip_mul_mat_prepare(members[0][0], k, dx.ptr, k, n, ws.ptr, wsz, None))
            self.check(self.lib.chip_mul_mat_group_run(arr, len(members), k, n, ws.ptr, wsz, None))
        else:
            self.check(self.lib.chip_mul_mat_group(arr, len(members), k, dx.ptr, k, n, ws.ptr, wsz, None))
        self.sync()
        res = [dy.download(np.float32, n * N).reshape(n, N) for dy, N in outs]
        if dh is not None:
            res.append(dh.download(np.uint16, outs[-1][1] * ld16).reshape(outs[-1][1], ld16))
        return res

    def mul_mat_group_rope(self, members, x, pos, ropes, freq_base=10000.0, check=True, norm=None):
        """chip_rope_table + chip_mul_mat_group_rope: members as mul_mat_group; ropes[i] = None or (head_dim, n_dims, mode,
        wants) with wants a subset of ("f32", "f16").  Returns (rc, list of dicts): a roped member's dict holds "f32" / "f16"
        arrays [n, N], an unroped member's "y".  norm = (weight row, eps): chip_mul_mat_group_rope_norm, and one more dict
        {"normed": [n, K]} at the end of the list."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        dx = self.to_device(x)
        dp = self.to_device(np.ascontiguousarray(pos, np.int32))
        arr = (Mat * len(members))()
        rp = (RopeAfter * len(members))()
        keep, outs = [], []
        wsz = 0
        for i, (wt, W) in enumerate(members):
            W = np.ascontiguousarray(W, np.uint8)
            N = W.shape[0]
            dW = self.to_device(W)
            keep.append(dW)
            wsz = max(wsz, self.lib.chip_mul_mat_workspace_size_n(wt, k, N, n))
            if ropes[i] is None:
                dy = self.alloc(n * N * 4)
                self.check(self.lib.chip_memset(dy.ptr, 0xFF, n * N * 4, None))
                arr[i] = Mat(wt, dW.ptr, self.row_size(wt, k), N, dy.ptr, N, None, 0)
                outs.append({"y": (dy, np.float32)})
                continue
            hd, n_dims, mode, wants = ropes[i]
            dt = self.alloc(n * n_dims * 4)
            self.check(self.lib.chip_rope_table(dp.ptr, None, n, n_dims, 4096, freq_base, 1.0, 0.0, 1.0, 32.0, 1.0, dt.ptr, None))
            keep.append(dt)
            o = {}
            if "f32" in wants:
                o["f32"] = (self.alloc(n * N * 4), np.float32)
                self.check(self.lib.chip_memset(o["f32"][0].ptr, 0xFF, n * N * 4, None))
            if "f16" in wants:
                o["f16"] = (self.alloc(n * N * 2), np.float16)
                self.check(self.lib.chip_memset(o["f16"][0].ptr, 0xFF, n * N * 2, None))
            arr[i] = Mat(wt, dW.ptr, self.row_size(wt, k), N, None, 0, None, 0)
            rp[i] = RopeAfter(dt.ptr, hd, n_dims, mode, o["f32"][0].ptr if "f32" in o else None, N, o["f16"][0].ptr if "f16" in o else None, N)
            outs.append(o)
        ws = self.alloc(max(wsz, 16))
        if norm is None:
            rc = self.lib.chip_mul_mat_group_rope(arr, rp, len(members), k, dx.ptr, k, n, ws.ptr, wsz, None)
        else:
            dw, dn = self.to_device(np.ascontiguousarray(norm[0], np.float32)), self.alloc(n * k * 4)
            self.check(self.lib.chip_memset(dn.ptr, 0xFF, n * k * 4, None))
            nb = NormBefore(dw.ptr, norm[1], dn.ptr, k)
            rc = self.lib.chip_mul_mat_group_rope_norm(arr, rp, C.byref(nb), len(members), k, dx.ptr, k, n, ws.ptr, wsz, None)
        if check:
            self.check(rc)
        self.sync()
        res = []
        for (wt, W), o in zip(members, outs):
            N = np.asarray(W).shape[0]
            res.append({key: buf.download(dt_, n * N).reshape(n, N) for key, (buf, dt_) in o.items()})
        if norm is not None:
            res.append({"normed": dn.download(np.float32, n * k).reshape(n, k)})
        return rc, res

    def mul_mat_pair(self, wtype, W1, W2, x):
        """Two matrices of one shape on the same activation (chip_mul_mat_pair): returns (y1, y2), each fp32 [n, N]."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        W1, W2 = np.ascontiguousarray(W1, np.uint8), np.ascontiguousarray(W2, np.uint8)
        N = W1.shape[0]
        nb01 = self.row_size(wtype, k)
        d1, d2, dx = self.to_device(W1), self.to_device(W2), self.to_device(x)
        y1, y2 = self.alloc(n * N * 4), self.alloc(n * N * 4)
        wsz = self.lib.chip_mul_mat_workspace_size_n(wtype, k, N, n)
        ws = self.alloc(wsz)
        self.check(self.lib.chip_mul_mat_pair(wtype, d1.ptr, d2.ptr, nb01, k, N, dx.ptr, k, n, y1.ptr, y2.ptr, N, ws.ptr, wsz, None))
        self.sync()
        return y1.download(np.float32, n * N).reshape(n, N), y2.download(np.float32, n * N).reshape(n, N)

    def mul_mat_pair_silu_mul(self, wtype, W1, W2, x, norm=None):
        """silu(W1 x) * (W2 x) in one launch (chip_mul_mat_pair_silu_mul): fp32 [n, N].  norm = (weight row, eps): the rows are
        normed in the prologue (chip_mul_mat_pair_silu_mul_norm) and (y, normed rows) is returned."""
        x = np.ascontiguousarray(x, np.float32)
        n, k = x.shape
        W1, W2 = np.ascontiguousarray(W1, np.uint8), np.ascontiguousarray(W2, np.uint8)
        N = W1.shape[0]
        nb01 = self.row_size(wtype, k)
        d1, d2, dx = self.to_device(W1), self.to_device(W2), self.to_device(x)
        y = self.alloc(n * N * 4)
        self.check(self.lib.chip_memset(y.ptr, 0xFF, n * N * 4, None))                   # NaN: unwritten rows show
        wsz = self.lib.chip_mul_mat_workspace_size_n(wtype, k, N, n)
        ws = self.alloc(wsz)
        if norm is not None:
            dw, dn = self.to_device(np.ascontiguousarray(norm[0], np.float32)), self.alloc(n * k * 4)
            self.check(self.lib.chip_memset(dn.ptr, 0xFF, n * k * 4, None))
            nb = NormBefore(dw.ptr, norm[1], dn.ptr, k)
            self.check(self.lib.chip_mul_mat_pair_silu_mul_norm(wtype, d1.ptr, d2.ptr, nb01, k, N, dx.ptr, k, n, C.byref(nb), y.ptr, N,
                                                                ws.ptr, wsz, None))
            self.sync()
            return y.download(np.float32, n * N).reshape(n, N), dn.download(np.float32, n * k).reshape(n, k)
        self.check(self.lib.chip_mul_mat_pair_silu_mul(wtype, d1.ptr, d2.ptr, nb01, k, N, dx.ptr, k, n, y.ptr, N, ws.ptr, wsz, None))
        self.sync()
        return y.download(np.float32, n * N).reshape(n, N)

    def mul_mat_add(self, wtype, W, x, addend, in_place=False):
        """W x + addend in one launch (chip_mul_mat_add): fp32 [n, N]; in_place: the result goes over the addend."""
        x, addend = np.ascontiguousarray(x, np.float32), np.ascontiguousarray(addend, np.float32)
        n, k = x.shape
        W = np.ascontiguousarray(W, np.uint8)
        N = W.shape[0]
        dW, dx, da = self.to_device(W), self.to_device(x), self.to_device(addend)
        y = da if in_place else self.alloc(n * N * 4)
        if not in_place:
            self.check(self.lib.chip_memset(y.ptr, 0xFF, n * N * 4, None))
        wsz = self.lib.chip_mul_mat_workspace_size_n(wtype, k, N, n)
        ws = self.alloc(wsz)
        self.check(self.lib.chip_mul_mat_add(wtype, dW.ptr, self.row_size(wtype, k), k, N, dx.ptr, k, n, da.ptr, N, y.ptr, N, ws.ptr, wsz, None))
        self.sync()
        return y.download(np.float32, n * N).reshape(n, N)

    def rms_norm_mul(self, x, w, eps):
        """chip_rms_norm_mul: the norm of every row times the weight row."""
        x = np.ascontiguousarray(x, np.float32)
        n, ne0 = x.shape
        dx, dw, dy = self.to_device(x), self.to_device(np.ascontiguousarray(w, np.float32)), self.alloc(x.nbytes)
        self.check(self.lib.chip_rms_norm_mul(dx.ptr, ne0, n, ne0, eps, dw.ptr, None, 0, dy.ptr, ne0, None))
        self.sync()
        return dy.download(np.float32, n * ne0).reshape(n, ne0)

    def rms_norm(self, x, eps):
        x = np.ascontiguousarray(x, np.float32)
        n, ne0 = x.shape
        dx, dy = self.to_device(x), self.alloc(x.nbytes)
        self.check(self.lib.chip_rms_norm(dx.ptr, ne0, n, ne0, eps, dy.ptr, ne0, None))
        self.sync()
        return dy.download(np.float32, n * ne0).reshape(n, ne0)

    def silu(self, x):
        x = np.ascontiguousarray(x, np.float32)
        n, ne0 = x.shape
        dx, dy = self.to_device(x), self.alloc(x.nbytes)
        self.check(self.lib.chip_silu(dx.ptr, ne0, n, ne0, dy.ptr, ne0, None))
        self.sync()
        return dy.download(np.float32, n * ne0).reshape(n, ne0)

    def silu_mul(self, a, b):
        """silu(a) * b in one launch (the FFN's gate * up)."""
        a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
        n, ne0 = a.shape
        da, db, dy = self.to_device(a), self.to_device(b), self.alloc(a.nbytes)
        self.check(self.lib.chip_silu_mul(da.ptr, ne0, db.ptr, ne0, n, ne0, dy.ptr, ne0, None))
        self.sync()
        return dy.download(np.float32, n * ne0).reshape(n, ne0)

    def binary(self, op, a, b):
        """op "add" or "mul"; b has the shape of a or is one row."""
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32).reshape(-1, a.shape[1])
        n, ne0 = a.shape
        da, db, dy = self.to_device(a), self.to_device(b), self.alloc(a.nbytes)
        fn = self.lib.chip_add if op == "add" else self.lib.chip_mul
        self.check(fn(da.ptr, ne0, db.ptr, ne0, b.shape[0], n, ne0, dy.ptr, ne0, None))
        self.sync()
        return dy.download(np.float32, n * ne0).reshape(n, ne0)

    # -- attention-side ops ---------------------------------------------------------------------------------
    def soft_max(self, x, mask=None, scale=1.0, max_bias=0.0):
        """x fp32 [n_head, ne01, ne00]; mask fp32 / fp16 [>= ne01, ne00] or None."""
        x = np.ascontiguousarray(x, np.float32)
        n_head, ne01, ne00 = x.shape
        dx, dy = self.to_device(x), self.alloc(x.nbytes)
        dm, mt = None, F32
        if mask is not None:
            mask = np.ascontiguousarray(mask)
            mt = F16 if mask.dtype == np.float16 else F32
            dm = self.to_device(mask)
        self.check(self.lib.chip_soft_max(dx.ptr, ne00, dm.ptr if dm else None, mt, ne00, ne01, n_head * ne01, scale, max_bias,
                                          dy.ptr, ne00, None))
        self.sync()
        return dy.download(np.float32, x.size).reshape(x.shape)

    def cpy(self, x, dst_dtype, dst_strides=None, dst_elems=None, dst_shape=None):
        """Copies the numpy array (or strided view) x, at most 4-D, into a destination of dst_dtype: dense (of x's shape,
        or of dst_shape with the same element count), or with the given byte strides (numpy order, slowest first) inside
        a zeroed region of dst_elems elements.  The source is uploaded with the view's own strides.  Returns the
        destination region as a flat array."""
        base = x
        while isinstance(base.base, np.ndarray):
            base = base.base
        base = np.ascontiguousarray(base) if not base.flags.c_contiguous else base
        off = x.__array_interface__["data"][0] - base.__array_interface__["data"][0]
        types = {np.dtype(np.float32): F32, np.dtype(np.float16): F16}
        dst_dtype = np.dtype(dst_dtype)
        pad = 4 - x.ndim
        ne = [1] * pad + list(x.shape)
        nbs = [0] * pad + list(x.strides)
        dshape = list(dst_shape if dst_shape is not None else x.shape)
        if dst_strides is None:
            dst_strides = list(np.empty(dshape, dst_dtype).strides)
            dst_elems = x.size
        ned = [1] * (4 - len(dshape)) + dshape
        nbd = [0] * (4 - len(dshape)) + list(dst_strides)
        A = C.c_int64 * 4
        dsrc = self.to_device(base.reshape(-1).view(np.uint8))
        ddst = self.alloc(dst_elems * dst_dtype.itemsize)
        ddst.upload(np.zeros(dst_elems * dst_dtype.itemsize, np.uint8))
        self.check(self.lib.chip_cpy(dsrc.ptr + off, types[x.dtype], A(*ne[::-1]), A(*nbs[::-1]), ddst.ptr, types[dst_dtype],
                                     A(*ned[::-1]), A(*nbd[::-1]), None))
        self.sync()
        return ddst.download(dst_dtype, dst_elems)

    def rope(self, x, pos, n_dims, mode, freq_factors=None, n_ctx_orig=4096, freq_base=10000.0, freq_scale=1.0,
             ext_factor=0.0, attn_factor=1.0, beta_fast=32.0, beta_slow=1.0, two_step=False, store_f16=False):
        """x fp32 [n_tokens, n_head, ne0], pos int32 [n_tokens].  two_step: chip_rope_table + chip_rope_apply.
        store_f16: chip_rope_table + chip_rope_apply_store; returns (y fp32, y fp16)."""
        x = np.ascontiguousarray(x, np.float32)
        ne2, ne1, ne0 = x.shape
        dx, dy = self.to_device(x), self.alloc(x.nbytes)
        dp = self.to_device(np.ascontiguousarray(pos, np.int32))
        df = self.to_device(np.ascontiguousarray(freq_factors, np.float32)) if freq_factors is not None else None
        if store_f16:
            dt, dh = self.alloc(ne2 * n_dims * 4), self.alloc(x.size * 2)
            self.check(self.lib.chip_rope_table(dp.ptr, df.ptr if df else None, ne2, n_dims, n_ctx_orig, freq_base, freq_scale,
                                                ext_factor, attn_factor, beta_fast, beta_slow, dt.ptr, None))
            self.check(self.lib.chip_rope_apply_store(dx.ptr, ne0, ne0 * ne1, dt.ptr, ne0, ne1, ne2, n_dims, mode, dy.ptr, ne0,
                                                      ne0 * ne1, dh.ptr, ne0, ne0 * ne1, None))
            self.sync()
            return dy.download(np.float32, x.size).reshape(x.shape), dh.download(np.float16, x.size).reshape(x.shape)
        if two_step:
            dt = self.alloc(ne2 * n_dims * 4)
            self.check(self.lib.chip_rope_table(dp.ptr, df.ptr if df else None, ne2, n_dims, n_ctx_orig, freq_base, freq_scale,
                                                ext_factor, attn_factor, beta_fast, beta_slow, dt.ptr, None))
            self.check(self.lib.chip_rope_apply(dx.ptr, ne0, ne0 * ne1, dt.ptr, ne0, ne1, ne2, n_dims, mode, dy.ptr, ne0, ne0 * ne1,
                                                None))
        else:
            self.check(self.lib.chip_rope(dx.ptr, ne0, ne0 * ne1, dp.ptr, df.ptr if df else None, ne0, ne1, ne2, n_dims, mode,
                                          n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow,
                                          dy.ptr, ne0, ne0 * ne1, None))
        self.sync()
        return dy.download(np.float32, x.size).reshape(x.shape)

    def rope_two(self, xa, xb, pos, n_dims, mode, want=(("f32",), ("f32", "f16")), freq_factors=None, n_ctx_orig=4096,
                 freq_base=10000.0, freq_scale=1.0, ext_factor=0.0, attn_factor=1.0, beta_fast=32.0, beta_slow=1.0):
        """chip_rope_table + chip_rope_apply_two: xa fp32 [n_tokens, heads_a, ne0], xb fp32 [n_tokens, heads_b, ne0] rotated in one
        launch; want names the outputs of each ("f32", "f16").  Returns ({"f32": .., "f16": ..}, {..}); outputs not asked
        for are absent."""
        xs = [np.ascontiguousarray(xa, np.float32), np.ascontiguousarray(xb, np.float32)]
        ne2, _, ne0 = xs[0].shape
        dp = self.to_device(np.ascontiguousarray(pos, np.int32))
        df = self.to_device(np.ascontiguousarray(freq_factors, np.float32)) if freq_factors is not None else None
        dt = self.alloc(ne2 * n_dims * 4)
        self.check(self.lib.chip_rope_table(dp.ptr, df.ptr if df else None, ne2, n_dims, n_ctx_orig, freq_base, freq_scale,
                                            ext_factor, attn_factor, beta_fast, beta_slow, dt.ptr, None))
        ops, bufs = [], []
        for x, w in zip(xs, want):
            ne1 = x.shape[1]
            dx = self.to_device(x)
            dy = self.alloc(x.nbytes) if "f32" in w else None
            dh = self.alloc(x.size * 2) if "f16" in w else None
            bufs.append((dx, dy, dh))
            ops.append(RopeOperand(dx.ptr, ne0, ne0 * ne1, ne1, dy.ptr if dy else None, ne0, ne0 * ne1, dh.ptr if dh else None, ne0,
                                   ne0 * ne1))
        self.check(self.lib.chip_rope_apply_two(C.byref(ops[0]), C.byref(ops[1]), dt.ptr, ne0, ne2, n_dims, mode, None))
        self.sync()
        out = []
        for x, (dx, dy, dh) in zip(xs, bufs):
            r = {}
            if dy:
                r["f32"] = dy.download(np.float32, x.size).reshape(x.shape)
            if dh:
                r["f16"] = dh.download(np.float16, x.size).reshape(x.shape)
            out.append(r)
        return tuple(out)

    def get_rows(self, t, table, nc, ids):
        """table uint8 [ne01, row_size(t, nc)] (or float32 / float16 [ne01, nc] for F32 / F16), ids int32 [n] -> fp32 [n, nc];
        rows of ids outside the table come back as NaN (left unwritten)."""
        table = np.ascontiguousarray(table)
        ids = np.ascontiguousarray(ids, np.int32)
        ne01 = table.shape[0]
        nb01 = table.strides[0]
        dt, di = self.to_device(table.reshape(-1).view(np.uint8)), self.to_device(ids)
        dy = self.alloc(max(ids.size * nc * 4, 16))
        self.check(self.lib.chip_memset(dy.ptr, 0xFF, max(ids.size * nc * 4, 16), None))
        self.check(self.lib.chip_get_rows(t, dt.ptr, nb01, nb01 * ne01, nb01 * ne01, nc, ne01, di.ptr, ids.size, 1, 1, ids.size,
                                          ids.size, dy.ptr, nc, nc * ids.size, nc * ids.size, None))
        self.sync()
        return dy.download(np.float32, ids.size * nc).reshape(ids.size, nc)

    def mul_mat_f16_batched(self, W, x, workspace=True, merged=False):
        """W fp16 array or view [ne02, N, K] (K contiguous), x fp32 array or view [ne12, n, K] (K contiguous) ->
        y fp32 [ne12, n, N]; the views are uploaded with their own strides.  workspace=False withholds the workspace
        (dot-product kernels only).  merged=True: chip_mul_mat_f16_batched_two_copies, returns (y, the second copy laid
        out [n, ne12 * N], a token's heads side by side)."""
        def upload(v):
            base = v
            while isinstance(base.base, np.ndarray):
                base = base.base
            assert base.flags.c_contiguous and v.strides[-1] == v.itemsize
            off = v.__array_interface__["data"][0] - base.__array_interface__["data"][0]
            return self.to_device(base.reshape(-1).view(np.uint8)), off
        ne02, N, K = W.shape
        ne12, n, _ = x.shape
        dw, woff = upload(W)
        dx, xoff = upload(x)
        dy = self.alloc(ne12 * n * N * 4)
        wsz = self.lib.chip_mul_mat_f16_batched_workspace_size(K, N, ne02, ne12, n) if workspace else 0
        ws = self.alloc(wsz) if wsz else None
        if merged:
            dy2 = self.alloc(ne12 * n * N * 4)
            self.check(self.lib.chip_memset(dy2.ptr, 0xFF, ne12 * n * N * 4, None))          # NaN: unwritten values show
            self.check(self.lib.chip_mul_mat_f16_batched_two_copies(dw.ptr + woff, W.strides[1], W.strides[0], K, N, ne02,
                                                                    dx.ptr + xoff, x.strides[1] // 4, x.strides[0] // 4, n, ne12,
                                                                    dy.ptr, N, n * N, dy2.ptr, ne12 * N, N, ws.ptr if ws else None,
                                                                    wsz, None))
            self.sync()
            return (dy.download(np.float32, ne12 * n * N).reshape(ne12, n, N), dy2.download(np.float32, ne12 * n * N).reshape(n, ne12 * N))
        self.check(self.lib.chip_mul_mat_f16_batched(dw.ptr + woff, W.strides[1], W.strides[0], K, N, ne02, dx.ptr + xoff,
                                                     x.strides[1] // 4, x.strides[0] // 4, n, ne12, dy.ptr, N, n * N,
                                                     ws.ptr if ws else None, wsz, None))
        self.sync()
        return dy.download(np.float32, ne12 * n * N).reshape(ne12, n, N)

    def mul_mat_id(self, wtype, W, x, ids):
        """LM_GGML_OP_MUL_MAT_ID: W uint8 [n_as, N, row_size], x fp32 [n_tokens, ne11, K], ids int32 [n_tokens, n_used]
        -> y [n_tokens, n_used, N]."""
        W = np.ascontiguousarray(W, np.uint8)
        x = np.ascontiguousarray(x, np.float32)
        ids = np.ascontiguousarray(ids, np.int32)
        n_tokens, ne11, k = x.shape
        n_as, N = W.shape[0], W.shape[1]
        n_used = ids.shape[1]
        nb01 = self.row_size(wtype, k)
        dW, dx, di = self.to_device(W), self.to_device(x), self.to_device(ids)
        dy = self.alloc(n_tokens * n_used * N * 4)
        self.check(self.lib.chip_memset(dy.ptr, 0xFF, max(n_tokens * n_used * N * 4, 16), None))   # NaN: unwritten rows show
        wsz = self.lib.chip_mul_mat_id_workspace_size(wtype, k, n_as, n_used, n_tokens, ne11)
        ws = self.alloc(wsz)
        self.check(self.lib.chip_mul_mat_id(wtype, dW.ptr, nb01, N * nb01, k, N, n_as, dx.ptr, k, ne11, di.ptr, n_used,
                                            n_used, n_tokens, dy.ptr, N, ws.ptr, wsz, None))
        self.sync()
        return dy.download(np.float32, n_tokens * n_used * N).reshape(n_tokens, n_used, N)

    def repack_q6_K(self, W, k, to_planes=True, in_place=False):
        """chip_repack_q6_K on a host matrix W uint8 [N, row_size(Q6_K, K)]: returns the repacked bytes."""
        W = np.ascontiguousarray(W, np.uint8)
        N, nb01 = W.shape
        src = self.to_device(W)
        dst = src if in_place else self.alloc(W.size)
        self.check(self.lib.chip_repack_q6_K(src.ptr, nb01, dst.ptr, nb01, k, N, 1 if to_planes else 0, None))
        self.sync()
        return dst.download(np.uint8, W.size).reshape(N, nb01)

    def block_isums(self, wtype, W, aq, k):
        """Per-block integer sums [n, N, K/block] (and imin for Q4_K / Q5_K) from reference-layout activation blocks."""
        W = np.ascontiguousarray(W, np.uint8)
        aq = np.ascontiguousarray(aq, np.uint8)
        N, n = W.shape[0], aq.shape[0]
        nblk = k // self.lib.chip_block_elems(wtype)
        dW, da = self.to_device(W), self.to_device(aq)
        di = self.alloc(n * N * nblk * 4)
        dm = self.alloc(n * N * nblk * 4)
        self.check(self.lib.chip_block_isums(wtype, dW.ptr, W.shape[1], k, N, da.ptr, n, di.ptr, dm.ptr, None))
        self.sync()
        isum = di.download(np.int32, n * N * nblk).reshape(n, N, nblk)
        imin = dm.download(np.int32, n * N * nblk).reshape(n, N, nblk) if wtype in (Q4_K, Q5_K) else None
        return isum, imin
