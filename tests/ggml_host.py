"""A minimal ggml host for backend tests: the reference's own ggml (oracle/_ref/libggml_ref.so, loaded
RTLD_GLOBAL so the backend resolves lm_ggml_* from it) driven through its public C API with ctypes.
This is what llama.cpp does with a backend: load it, allocate weights in its buffer type, build a graph with
lm_ggml_mul_mat, let the scheduler split it, compute, read the result back."""
import ctypes as C
import os

import numpy as np

import oracle as O

vp, i64, i32, sz = C.c_void_p, C.c_int64, C.c_int, C.c_size_t
EVAL_CB = C.CFUNCTYPE(C.c_bool, C.c_int, vp, vp, vp)


class DevCaps(C.Structure):
    _fields_ = [("async_", C.c_bool), ("host_buffer", C.c_bool), ("buffer_from_host_ptr", C.c_bool), ("events", C.c_bool)]


class DevProps(C.Structure):            # struct lm_ggml_backend_dev_props (reference ggml-backend.h:152-159)
    _fields_ = [("name", C.c_char_p), ("description", C.c_char_p), ("memory_free", C.c_size_t),
                ("memory_total", C.c_size_t), ("type", C.c_int), ("caps", DevCaps)]


class Host:
    def __init__(self):
        self.ref = O.Reference()                       # RTLD_GLOBAL, fp16 table initialised
        self.L = L = self.ref.lib
        L.lm_ggml_backend_load.restype = vp
        L.lm_ggml_backend_load.argtypes = [C.c_char_p]
        L.lm_ggml_backend_reg_name.restype = C.c_char_p
        L.lm_ggml_backend_reg_name.argtypes = [vp]
        L.lm_ggml_backend_reg_dev_count.restype = sz
        L.lm_ggml_backend_reg_dev_count.argtypes = [vp]
        L.lm_ggml_backend_reg_dev_get.restype = vp
        L.lm_ggml_backend_reg_dev_get.argtypes = [vp, sz]
        L.lm_ggml_backend_reg_by_name.restype = vp
        L.lm_ggml_backend_reg_by_name.argtypes = [C.c_char_p]
        L.lm_ggml_backend_dev_name.restype = C.c_char_p
        L.lm_ggml_backend_dev_name.argtypes = [vp]
        L.lm_ggml_backend_dev_description.restype = C.c_char_p
        L.lm_ggml_backend_dev_description.argtypes = [vp]
        L.lm_ggml_backend_dev_type.restype = i32
        L.lm_ggml_backend_dev_type.argtypes = [vp]
        L.lm_ggml_backend_dev_memory.argtypes = [vp, C.POINTER(sz), C.POINTER(sz)]
        L.lm_ggml_backend_dev_init.restype = vp
        L.lm_ggml_backend_dev_init.argtypes = [vp, C.c_char_p]
        L.lm_ggml_backend_dev_buffer_type.restype = vp
        L.lm_ggml_backend_dev_buffer_type.argtypes = [vp]
        L.lm_ggml_backend_dev_supports_op.restype = C.c_bool
        L.lm_ggml_backend_dev_supports_op.argtypes = [vp, vp]
        L.lm_ggml_backend_dev_supports_buft.restype = C.c_bool
        L.lm_ggml_backend_dev_supports_buft.argtypes = [vp, vp]
        L.lm_ggml_backend_name.restype = C.c_char_p
        L.lm_ggml_backend_name.argtypes = [vp]
        L.lm_ggml_backend_get_default_buffer_type.restype = vp
        L.lm_ggml_backend_get_default_buffer_type.argtypes = [vp]
        L.lm_ggml_backend_buft_name.restype = C.c_char_p
        L.lm_ggml_backend_buft_name.argtypes = [vp]
        L.lm_ggml_backend_buft_is_host.restype = C.c_bool
        L.lm_ggml_backend_buft_is_host.argtypes = [vp]
        L.lm_ggml_backend_alloc_ctx_tensors_from_buft.restype = vp
        L.lm_ggml_backend_alloc_ctx_tensors_from_buft.argtypes = [vp, vp]
        L.lm_ggml_backend_buffer_set_usage.argtypes = [vp, i32]
        L.lm_ggml_backend_buffer_get_size.restype = sz
        L.lm_ggml_backend_buffer_get_size.argtypes = [vp]
        L.lm_ggml_backend_buffer_clear.argtypes = [vp, C.c_uint8]
        L.lm_ggml_backend_tensor_memset.argtypes = [vp, C.c_uint8, sz, sz]
        L.lm_ggml_backend_tensor_copy.argtypes = [vp, vp]
        L.lm_ggml_backend_synchronize.argtypes = [vp]
        L.lm_ggml_backend_sched_new.restype = vp
        L.lm_ggml_backend_sched_new.argtypes = [C.POINTER(vp), C.POINTER(vp), i32, sz, C.c_bool, C.c_bool]
        L.lm_ggml_backend_sched_free.argtypes = [vp]
        L.lm_ggml_backend_sched_alloc_graph.restype = C.c_bool
        L.lm_ggml_backend_sched_alloc_graph.argtypes = [vp, vp]
        L.lm_ggml_backend_sched_graph_compute.restype = i32
        L.lm_ggml_backend_sched_graph_compute.argtypes = [vp, vp]
        L.lm_ggml_backend_sched_get_n_splits.restype = i32
        L.lm_ggml_backend_sched_get_n_splits.argtypes = [vp]
        L.lm_ggml_backend_sched_get_tensor_backend.restype = vp
        L.lm_ggml_backend_sched_get_tensor_backend.argtypes = [vp, vp]
        L.lm_ggml_backend_sched_reset.argtypes = [vp]
        L.lm_ggml_backend_sched_set_tensor_backend.argtypes = [vp, vp, vp]
        L.lm_ggml_backend_compare_graph_backend.restype = C.c_bool
        L.lm_ggml_backend_compare_graph_backend.argtypes = [vp, vp, vp, EVAL_CB, vp]
        L.lm_ggml_backend_dev_get_props.argtypes = [vp, C.POINTER(DevProps)]
        L.lm_ggml_backend_dev_host_buffer_type.restype = vp
        L.lm_ggml_backend_dev_host_buffer_type.argtypes = [vp]
        L.lm_ggml_backend_buft_alloc_buffer.restype = vp
        L.lm_ggml_backend_buft_alloc_buffer.argtypes = [vp, sz]
        L.lm_ggml_backend_buft_get_device.restype = vp
        L.lm_ggml_backend_buft_get_device.argtypes = [vp]
        L.lm_ggml_backend_buffer_get_base.restype = vp
        L.lm_ggml_backend_buffer_get_base.argtypes = [vp]
        L.lm_ggml_backend_buffer_get_type.restype = vp
        L.lm_ggml_backend_buffer_get_type.argtypes = [vp]
        L.lm_ggml_backend_buffer_is_host.restype = C.c_bool
        L.lm_ggml_backend_buffer_is_host.argtypes = [vp]
        L.lm_ggml_backend_event_new.restype = vp
        L.lm_ggml_backend_event_new.argtypes = [vp]
        L.lm_ggml_backend_event_free.argtypes = [vp]
        L.lm_ggml_backend_event_record.argtypes = [vp, vp]
        L.lm_ggml_backend_event_synchronize.argtypes = [vp]
        L.lm_ggml_backend_event_wait.argtypes = [vp, vp]
        L.lm_ggml_backend_tensor_set_async.argtypes = [vp, vp, vp, sz, sz]
        L.lm_ggml_backend_tensor_get_async.argtypes = [vp, vp, vp, sz, sz]
        L.lm_ggml_add.restype = vp
        L.lm_ggml_add.argtypes = [vp, vp, vp]
        L.lm_ggml_mul.restype = vp
        L.lm_ggml_mul.argtypes = [vp, vp, vp]
        L.lm_ggml_silu.restype = vp
        L.lm_ggml_silu.argtypes = [vp, vp]
        L.lm_ggml_rms_norm.restype = vp
        L.lm_ggml_rms_norm.argtypes = [vp, vp, C.c_float]
        L.lm_ggml_soft_max.restype = vp
        L.lm_ggml_soft_max.argtypes = [vp, vp]
        L.lm_ggml_sqr.restype = vp
        L.lm_ggml_sqr.argtypes = [vp, vp]
        L.lm_ggml_new_tensor_1d.restype = vp
        L.lm_ggml_new_tensor_1d.argtypes = [vp, i32, i64]
        L.lm_ggml_set_name.restype = vp
        L.lm_ggml_set_name.argtypes = [vp, C.c_char_p]
        L.lm_ggml_set_input.argtypes = [vp]
        L.lm_ggml_set_output.argtypes = [vp]
        L.lm_ggml_nbytes.restype = sz
        L.lm_ggml_nbytes.argtypes = [vp]
        L.lm_ggml_reshape_2d.restype = vp
        L.lm_ggml_reshape_2d.argtypes = [vp, vp, i64, i64]
        L.lm_ggml_reshape_3d.restype = vp
        L.lm_ggml_reshape_3d.argtypes = [vp, vp, i64, i64, i64]
        L.lm_ggml_view_1d.restype = vp
        L.lm_ggml_view_1d.argtypes = [vp, vp, i64, sz]
        L.lm_ggml_view_3d.restype = vp
        L.lm_ggml_view_3d.argtypes = [vp, vp, i64, i64, i64, sz, sz, sz]
        L.lm_ggml_cont_2d.restype = vp
        L.lm_ggml_cont_2d.argtypes = [vp, vp, i64, i64]

    def context(self, n_tensors=32, with_graph=True):
        L = self.L
        size = L.lm_ggml_tensor_overhead() * n_tensors + (L.lm_ggml_graph_overhead() if with_graph else 0) + 4096
        return L.lm_ggml_init(O._InitParams(size, None, True))

    def tensor_2d(self, ctx, t, ne0, ne1, name=None):
        p = self.L.lm_ggml_new_tensor_2d(ctx, t, ne0, ne1)
        if name:
            self.L.lm_ggml_set_name(p, name.encode())
        return p

    def tensor_3d(self, ctx, t, ne0, ne1, ne2, name=None):
        p = self.L.lm_ggml_new_tensor_3d(ctx, t, ne0, ne1, ne2)
        if name:
            self.L.lm_ggml_set_name(p, name.encode())
        return p

    def set(self, tensor, arr):
        arr = np.ascontiguousarray(arr)
        self.L.lm_ggml_backend_tensor_set(tensor, arr.ctypes.data_as(vp), 0, arr.nbytes)

    def get(self, tensor, dtype, shape):
        out = np.empty(shape, dtype)
        self.L.lm_ggml_backend_tensor_get(tensor, out.ctypes.data_as(vp), 0, out.nbytes)
        return out

    def load_hip(self):
        import cactus_amd
        reg = self.L.lm_ggml_backend_load(cactus_amd.BACKEND_LIB.encode())
        assert reg, "lm_ggml_backend_load(libggml-hip.so) returned NULL"
        return reg
