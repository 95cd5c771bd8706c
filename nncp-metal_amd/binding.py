"""ctypes binding of the libnc-compatible C ABI (include/nc_api.h, nc_ext.h).

The same binding drives either shared library that exports the ABI; the
product is csrc/libnc_hip.so.  Tensors cross the boundary as numpy arrays:
libnc is column-major (dims[0] contiguous), so a libnc tensor of dims
(d0, d1, d2) is a C-contiguous numpy array of shape (d2, d1, d0).
"""
import ctypes as C
import os
import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIB = os.path.join(HERE, "csrc", "libnc_hip.so")

# NCTypeEnum (libnc.h:80-98)
F32, BF16, F16, I8, I16, I32, U8, U16, U32 = range(9)
_NP = {F32: np.float32, I8: np.int8, I32: np.int32, U16: np.uint16, U8: np.uint8}
_NC = {np.dtype(v): k for k, v in _NP.items()}
_NP[BF16] = np.uint16      # read as its 16 bits; numpy() widens them to float32


def bf16_bits(a):
    """float32 array -> the 16 bits of each value rounded to bf16 (nearest even)"""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16).reshape(np.shape(a))


def bf16_widen(bits):
    """the float32 value of each 16-bit bf16 pattern"""
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(bits))

SGD_OPT_BASIC, SGD_OPT_ADAM, SGD_OPT_RMSPROP = 0, 1, 16
NC_PAD_ZERO, NC_PAD_DUP = 0, 1
ACT_NONE, ACT_GELU, ACT_RELU = 0, 1, 2


class SGDOptParams(C.Structure):
    """libnc.h:546-559"""
    _fields_ = [("algo", C.c_int), ("beta1", C.c_float), ("beta2", C.c_float),
                ("eps", C.c_float), ("gradient_clip", C.c_float),
                ("weight_decay", C.c_float), ("loss_scale", C.c_float),
                ("lr", C.c_float)]


class ListHead(C.Structure):
    pass


ListHead._fields_ = [("prev", C.POINTER(ListHead)), ("next", C.POINTER(ListHead))]


class NCParamList(C.Structure):
    """libnc.h:512-516"""
    _fields_ = [("ctx", C.c_void_p), ("param_list", ListHead), ("add_graph", C.c_int)]


PARAM_UPDATE_FUNC = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, C.c_void_p)

_P = C.c_void_p
_SZ = C.c_size_t
_SSZ = C.c_ssize_t
_I = C.c_int
_F = C.c_float

# name: (restype, argtypes)
_PROTOS = {
    "nc_context_init": (_P, [_I]), "nc_context_end": (None, [_P]),
    "nc_new_cpu_device": (_P, [_P]), "nc_new_cuda_device": (_P, [_P, _I]),
    "nc_synchronize": (None, [_P]),
    "nc_new_tensor": (_P, [_P, _I, _I, C.POINTER(_SZ)]),
    "nc_new_tensor_nz": (_P, [_P, _I, _I, C.POINTER(_SZ)]),
    "nc_new_tensor_2d": (_P, [_P, _I, _SZ, _SZ]),
    "nc_new_f32": (_P, [_P, _F]),
    "nc_dup_tensor": (_P, [_P]), "nc_free_tensor": (None, [_P]),
    "nc_tensor_get_hash": (C.c_uint32, [_P]),
    "nc_get_node": (_P, [_P]), "nc_tensor_get_item_type": (_I, [_P]),
    "nc_tensor_get_ptr": (_P, [_P, C.POINTER(_SZ)]),
    "nc_tensor_get_dims": (_I, [_P, C.POINTER(_SZ)]),
    "nc_tensor_set_zero": (None, [_P]), "nc_tensor_set_f32": (None, [_P, _F]),
    "nc_rnd_init": (_P, [_P, C.c_uint32]), "nc_rnd_end": (None, [_P]),
    "nc_tensor_set_rnd_unif": (None, [_P, _F, _F, _P]),
    "nc_tensor_set_dropout": (None, [_P, _F, _P]),
    "nc_set1_i32_2d": (None, [_P, _SZ, _SZ, C.c_int32]),
    "nc_get_scalar_f32": (_F, [_P]),
    "nc_tensor_copy": (None, [_P, _P]),
    "nc_tensor_copy_slice": (None, [_P, _P, _I, _SZ, _SZ, _SZ]),
    "nc_tensor_to_device": (_P, [_P, _P]), "nc_tensor_to_cpu_device": (_P, [_P]),
    "nc_get_tensor_device": (_P, [_P]),
    "nc_convert": (_P, [_P, _I]), "nc_add": (_P, [_P, _P]), "nc_mul": (_P, [_P, _P]),
    "nc_masked_fill": (_P, [_P, _P, _F, _I]),
    "nc_sigmoid": (_P, [_P]), "nc_tanh": (_P, [_P]), "nc_relu": (_P, [_P]),
    "nc_gelu": (_P, [_P]), "nc_gated_swish": (_P, [_P, _P, _F]),
    "nc_lstm_clamped": (_P, [_P, _P, _P, _P]), "nc_lerp": (_P, [_P, _P, _P]),
    "nc_reshape_1d": (_P, [_P, _SZ]), "nc_reshape_2d": (_P, [_P, _SZ, _SZ]),
    "nc_reshape_3d": (_P, [_P, _SZ, _SZ, _SZ]),
    "nc_reshape_4d": (_P, [_P, _SZ, _SZ, _SZ, _SZ]),
    "nc_repeat_1d": (_P, [_P, _SZ]), "nc_repeat_2d": (_P, [_P, _SZ, _SZ]),
    "nc_reduce_sum": (_P, [_P, _P, _I]), "nc_sum": (_P, [_P]),
    "nc_slice_alias": (_P, [_P, _I, _SZ, _SZ]), "nc_slice": (_P, [_P, _I, _SZ, _SZ]),
    "nc_concat": (_P, [C.POINTER(_P), _I, _I]),
    "nc_split": (None, [C.POINTER(_P), _P, _I, C.POINTER(_SZ), _I]),
    "nc_pad": (_P, [_P, _SSZ, _I, _SSZ, _I]),
    "nc_permute": (_P, [_P, _I, C.POINTER(_I)]),
    "nc_permute_4d": (_P, [_P, _I, _I, _I, _I]),
    "nc_matmul_add": (_P, [_P, _P, _P, _I, _I, _F]), "nc_matmul": (_P, [_P, _P]),
    "nc_get_col": (_P, [_P, _P]), "nc_soft_max": (_P, [_P]),
    "nc_indexed_log": (_P, [_P, _P]),
    "nc_layer_norm": (_P, [_P, _F]), "nc_rms_norm": (_P, [_P, _F]),
    "nc_fused_layer_norm": (_P, [_P, _P, _P, _F, _I]),
    "nc_rel_shift": (_P, [_P, _SSZ, _SSZ]),
    "nc_set_param": (_P, [_P, _P]),
    "nc_dup_node": (_P, [_P]), "nc_free_node": (None, [_P]),
    "nc_concat_node": (_P, [_P, C.POINTER(_P), _I, _I, C.POINTER(_SZ)]),
    "nc_concat_optimization": (None, [_P, C.POINTER(_P), _I]),
    "nc_node_set_parent": (None, [_P, _I, _P]), "nc_node_set_arg": (None, [_P, _I, _P]),
    "nc_backward": (None, [_P, _P, PARAM_UPDATE_FUNC, _I]),
    "nc_param_list_init": (None, [_P, C.POINTER(NCParamList)]),
    "nc_param_list_end": (None, [C.POINTER(NCParamList)]),
    "nc_get_param_count": (_SZ, [C.POINTER(NCParamList)]),
    "nc_sgd_opt_init": (_P, [_P, C.POINTER(SGDOptParams)]),
    "nc_sgd_opt_end": (None, [_P]),
    "sgd_opt_update_var": (None, [_P, _P, _P]),
    "nc_sgd_opt_set_all": (None, [C.POINTER(NCParamList), _P]),
    "nc_sgd_opt_update": (None, [_P]), "nc_sgd_opt_set_lr": (None, [_P, _F]),
    "vec_sum_f32": (_F, [C.POINTER(_F), _SZ]),
    # nc_ext.h
    "nc_linear": (_P, [_P, _P, _P, _I]),
    "nc_linear_add": (_P, [_P, _P, _P, _I, _P]),
    "nc_relpos_attention_step": (_P, [_P, _P, _P, _P, _P, _I, _I, _I, C.c_float, _I]),
    "nc_keep_k_major_weight": (None, [_P]), "nc_forget_k_major_weights": (None, [_P]),
    "nc_norm_linear_pair_into": (_P, [_P, _P, _P, C.c_float, _I, _P, _P, _I, _P, _P, _I, C.POINTER(_P)]),
    "nc_linear_pair_into": (_P, [_P, _P, _P, _P, _P, _I]),
    "nc_set_matmul_width_invariant": (_I, [_P, _I]),
    "nc_relpos_attention": (_P, [_P, _P, _P, _P, _P, _I, _I, _I, _F]),
    "nc_soft_max_int": (_P, [_P, C.c_float]),
    "nc_soft_max_cdf16": (_P, [_P]), "nc_cdf_lookup": (_P, [_P, _P]), "nc_cdf_path": (_P, [_P, _P]), "nc_soft_max_cdf16_path": (_P, [_P, _P]), "nc_soft_max_cdf16_path_to_host": (_P, [_P, _P]),
    "nc_tensor_to_cpu_device_queued": (_P, [_P]),
    "nc_soft_max_cdf16_to_host": (_P, [_P]), "nc_get_col_host_indices": (_P, [_P, _P, C.c_float]),
    "nc_exp_det": (_F, [_F]),
    "nc_set_matmul_bf16": (_I, [_P, _I]),
    "nc_get_launch_count": (C.c_int64, [_P]),
    "nc_get_bf16_cast_count": (C.c_int64, [_P]), "nc_set_bf16_shadow_check": (_I, [_I]),
    "nc_set_bf16_copy_of_results": (_I, [_P, _I]),
    "nc_context_stream": (_P, [_P]),
    "nc_set_deferred_weight_grad": (_I, [_P, _I]),
}
# variadic: bound without argtypes
_VARIADIC = ["nc_new_param", "nc_tensor_set_name"]

EXPORTED = sorted(list(_PROTOS) + _VARIADIC + [
    "nc_malloc", "nc_mallocz", "nc_free", "nc_new_device", "nc_prof_dump",
    "nc_new_tensor_from_tensor_nz", "nc_new_scalar", "nc_new_tensor_1d",
    "nc_new_tensor_3d", "nc_new_tensor_4d", "nc_vconcat", "nc_hconcat",
    "nc_cmul", "nc_combine_nodes"])


class NC:
    """One loaded library + one context with a host and a compute device."""

    def __init__(self, libpath=HIP_LIB, use_device=True, nb_threads=1):
        if not os.path.exists(libpath):
            raise RuntimeError(
                "%s is missing: build it first (python -c 'import __graft_entry__ as g; "
                "g.build()'); there is no fallback path" % libpath)
        self.lib = C.CDLL(libpath, mode=C.RTLD_LOCAL)
        for name, (res, args) in _PROTOS.items():
            f = getattr(self.lib, name)
            f.restype, f.argtypes = res, args
        self.lib.nc_new_param.restype = _P
        self.ctx = self.lib.nc_context_init(nb_threads)
        self.cpu = self.lib.nc_new_cpu_device(self.ctx)
        self.dev = self.lib.nc_new_cuda_device(self.ctx, 0) if use_device else self.cpu
        self._keep = []

    def __getattr__(self, name):
        if name.startswith("nc_") or name in ("sgd_opt_update_var", "vec_sum_f32"):
            return getattr(self.lib, name)
        raise AttributeError(name)

    # ---- numpy <-> tensor ------------------------------------------------
    def tensor(self, arr, device=None):
        """Owned tensor holding a copy of arr (see module docstring for axes)."""
        arr = np.asarray(arr)
        if not arr.flags.c_contiguous:
            arr = arr.copy(order="C")
        t = _NC[arr.dtype]
        dims = (_SZ * max(arr.ndim, 1))(*reversed(arr.shape))
        x = self.lib.nc_new_tensor_nz(self.cpu, t, arr.ndim, dims)
        ptr = self.lib.nc_tensor_get_ptr(x, None)
        C.memmove(ptr, arr.ctypes.data, arr.nbytes)
        return self.lib.nc_tensor_to_device(x, self.dev if device is None else device)

    def dims(self, x):
        d = (_SZ * 8)()
        n = self.lib.nc_tensor_get_dims(x, d)
        return tuple(d[i] for i in range(n))

    def numpy(self, x, free=False):
        """Copy of tensor x as a numpy array; x is borrowed unless free=True."""
        dims = self.dims(x)
        t = self.lib.nc_tensor_get_item_type(x)
        h = self.lib.nc_tensor_to_cpu_device(self.lib.nc_dup_tensor(x))
        n = int(np.prod(dims)) if dims else 1
        ptr = self.lib.nc_tensor_get_ptr(h, None)
        buf = (C.c_char * (n * np.dtype(_NP[t]).itemsize)).from_address(ptr)
        out = np.frombuffer(buf, dtype=_NP[t]).copy().reshape(tuple(reversed(dims)))
        if t == BF16:
            out = bf16_widen(out)
        self.lib.nc_free_tensor(h)
        if free:
            self.lib.nc_free_tensor(x)
        return out

    def dup(self, x):
        return self.lib.nc_dup_tensor(x)

    def free(self, *xs):
        for x in xs:
            self.lib.nc_free_tensor(x)

    # ---- parameters and gradients ---------------------------------------
    def param(self, arr, name="p"):
        """Parameter leaf; returns (holder, tensor): holder keeps the NCTensor*
        slot whose address the library records (libnc.h:503)."""
        holder = _P(self.tensor(arr))
        if not hasattr(self, "plist"):
            self.plist = NCParamList()
            self.lib.nc_param_list_init(self.ctx, C.byref(self.plist))
        p = self.lib.nc_new_param(C.byref(self.plist), C.byref(holder), name.encode())
        self._keep.append(holder)
        return holder, p

    def backward(self, y, grad=None):
        """Runs nc_backward on y (borrowed) and returns {param_ptr: ndarray}."""
        grads = {}

        def cb(opaque, g, idx):
            a = self.numpy(g, free=True)
            grads[opaque] = grads[opaque] + a if opaque in grads else a

        fn = PARAM_UPDATE_FUNC(cb)
        g = self.lib.nc_new_f32(self.dev, 1.0) if grad is None else grad
        self.lib.nc_backward(y, g, fn, 0)
        return grads

    def close(self):
        if hasattr(self, "plist"):
            self.lib.nc_param_list_end(C.byref(self.plist))
            del self.plist
        self.lib.nc_context_end(self.ctx)
