"""ctypes binding of the host side (include/nncp_host.h): the Transformer-XL
model class of nncp.c, the block loop and the coders, linked against
csrc/libnc_hip.so in host/libnncp_host_hip.so."""
import ctypes as C
import os

import numpy as np

from . import binding as B

HERE = os.path.dirname(os.path.abspath(__file__))
HOST_HIP_LIB = os.path.join(HERE, "host", "libnncp_host_hip.so")

MODE_SEQ_EVAL, MODE_SEGMENT, MODE_STEP_DECODE = 0, 1, 4
CODER_FLOAT, CODER_CDF16 = 0, 2
LN_POST, LN_PRE, LN_FINAL, LN_COEF, LN_RMSNORM = 1, 2, 4, 8, 16
FF_RELU, FF_GELU, FF_GEGLU, FF_GATED_SILU = 0, 1, 2, 3


class NNCPInterp(C.Structure):
    _fields_ = [("n_steps", C.c_int), ("val", C.c_float * 9), ("pos", C.c_int64 * 8),
                ("decay_power", C.c_float)]


class NNCPConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("n_layer", "d_model", "n_head", "d_key", "d_value",
                                       "d_inner", "d_pos", "mem_len")] + \
               [("attn_len", C.c_int * 32)] + \
               [(n, C.c_int) for n in ("use_bias", "use_w_r", "tied_w_r", "tied_b_r", "query_bias",
                                       "ln_flags", "ff_act")] + \
               [("init_range", C.c_float), ("embed_mult", C.c_float), ("sgd_opt", B.SGDOptParams)] + \
               [(n, C.c_int) for n in ("batch_size", "seg_len", "n_symbols")] + \
               [("seed", C.c_uint32), ("use_device", C.c_int), ("fused", C.c_int), ("nb_threads", C.c_int)] + \
               [("dropout_prob", C.c_float), ("dropout_att_prob", C.c_float), ("retrain_period", C.c_int),
                ("retrain_len", C.c_int), ("has_retrain_lr", C.c_int), ("retrain_lr", NNCPInterp)] + \
               [(n, C.c_int) for n in ("model_type", "lstm_n_cells", "lstm_n_cells2", "lstm_n_embed_out",
                                       "lstm_type", "lstm_full_connect", "lstm_use_layer_norm")] + \
               [("lstm_forget_bias", C.c_float), ("param_bf16", C.c_int)]


class NNCPStats(C.Structure):
    _fields_ = [("n_symbols", C.c_int64), ("n_steps", C.c_int64), ("loss_bits", C.c_double),
                ("t_eval", C.c_double), ("t_code", C.c_double), ("t_grad", C.c_double),
                ("t_update", C.c_double)]


class NNCPPutBit(C.Structure):
    _fields_ = [("range", C.c_uint32), ("low", C.c_uint32), ("current_byte", C.c_uint8),
                ("n_bytes", C.c_uint32), ("buf", C.c_void_p), ("buf_size", C.c_size_t),
                ("idx", C.c_size_t), ("overflow", C.c_int), ("sink", C.c_void_p),
                ("sink_opaque", C.c_void_p), ("n_flushed", C.c_size_t)]


class NNCPGetBit(C.Structure):
    _fields_ = [("buf", C.c_void_p), ("buf_len", C.c_size_t), ("idx", C.c_size_t),
                ("low", C.c_uint32), ("range", C.c_uint32)]


class NNCPFileParams(C.Structure):
    _fields_ = [("lr", NNCPInterp), ("block_len", NNCPInterp), ("use_bf16", C.c_int),
                ("max_size", C.c_int64), ("mode", C.c_int)]


MODEL_TRF, MODEL_LSTM = 0, 1
LSTM_NORMAL, LSTM_CLAMPED, LSTM_TIED = 0, 1, 2


def make_lstm_config(**kw):
    """nncp's "lstm" profile (nncp.c:2574-2603) with overrides."""
    cfg = NNCPConfig()
    opt = kw.pop("sgd_opt", None)
    base = dict(model_type=MODEL_LSTM, n_layer=4, lstm_n_cells=352, lstm_type=LSTM_CLAMPED, lstm_full_connect=1,
                lstm_use_layer_norm=1, lstm_forget_bias=0.0, batch_size=32, seg_len=20, n_symbols=256, seed=123,
                use_device=1, nb_threads=1)
    base.update(kw)
    base.setdefault("lstm_n_cells2", base["lstm_n_cells"])
    base.setdefault("lstm_n_embed_out", base["n_layer"])
    for k, v in base.items():
        setattr(cfg, k, v)
    cfg.sgd_opt = opt if opt is not None else B.SGDOptParams(
        algo=B.SGD_OPT_ADAM, beta1=0.0, beta2=0.9999, eps=1e-10, gradient_clip=0.0, lr=4e-3)
    return cfg


def constant_lr(lr):
    p = NNCPInterp()
    p.n_steps = 0
    p.val[0] = lr
    return p


def make_config(**kw):
    """nncp's default profile (nncp.c:2471-2513) with overrides; d_key/d_value
    follow d_model / n_head and attn_len defaults to mem_len + seg_len."""
    cfg = NNCPConfig()
    opt = kw.pop("sgd_opt", None)
    attn = kw.pop("attn_len", None)
    retrain_lr = kw.pop("retrain_lr", None)
    base = dict(n_layer=4, d_model=256, n_head=8, d_inner=512, d_pos=32, mem_len=32, use_bias=1,
                use_w_r=1, tied_w_r=1, tied_b_r=1, query_bias=0, ln_flags=LN_POST, ff_act=FF_GELU,
                init_range=1.0, embed_mult=1.0, batch_size=16, seg_len=32, n_symbols=256, seed=123,
                use_device=1, fused=0, nb_threads=1)
    base.update(kw)
    base.setdefault("d_key", base["d_model"] // base["n_head"])
    base.setdefault("d_value", base["d_key"])
    for k, v in base.items():
        setattr(cfg, k, v)
    for i in range(base["n_layer"]):
        cfg.attn_len[i] = (attn[i] if attn else base["mem_len"] + base["seg_len"])
    if retrain_lr is not None:
        cfg.has_retrain_lr = 1
        cfg.retrain_lr = retrain_lr if isinstance(retrain_lr, NNCPInterp) else constant_lr(retrain_lr)
    cfg.sgd_opt = opt if opt is not None else B.SGDOptParams(
        algo=B.SGD_OPT_ADAM, beta1=0.0, beta2=0.9999, eps=1e-8, gradient_clip=0.1, lr=3e-4)
    return cfg


_P = C.c_void_p


class Host:
    """Loaded host library; its libnc functions come from the libnc it links."""

    def __init__(self, libpath=HOST_HIP_LIB, nc_libpath=B.HIP_LIB):
        for p in (libpath, nc_libpath):
            if not os.path.exists(p):
                raise RuntimeError("%s is missing: run __graft_entry__.build() first" % p)
        # the libnc dependency is found through the rpath recorded at link time
        self.lib = C.CDLL(libpath, mode=C.RTLD_LOCAL)
        L = self.lib
        L.nncp_model_new.restype = _P
        L.nncp_model_new.argtypes = [C.POINTER(NNCPConfig)]
        L.nncp_model_free.argtypes = [_P]
        for n in ("nncp_model_context", "nncp_model_device", "nncp_model_cpu_device"):
            getattr(L, n).restype = _P
            getattr(L, n).argtypes = [_P]
        L.nncp_model_param.restype = C.POINTER(_P)
        L.nncp_model_param.argtypes = [_P, C.c_char_p]
        L.nncp_model_param_count.argtypes = [_P]
        L.nncp_model_opt_state.restype = _P
        L.nncp_model_opt_state.argtypes = [_P, C.c_char_p, C.c_int]
        L.nncp_model_set_opt_state.argtypes = [_P, C.c_char_p, C.c_int, _P]
        L.nncp_model_memory.restype = _P
        L.nncp_model_memory.argtypes = [_P, C.c_int]
        L.nncp_model_param_name.restype = C.c_char_p
        L.nncp_model_param_name.argtypes = [_P, C.c_int]
        for n in ("nncp_model_save_coefs", "nncp_model_load_coefs"):
            getattr(L, n).restype = None
            getattr(L, n).argtypes = [_P, C.c_char_p]
        L.nncp_model_train_step.restype = C.c_int64
        L.nncp_model_train_step.argtypes = [_P]
        L.trf_eval.restype = _P
        L.trf_eval.argtypes = [_P, C.c_int, _P]
        L.trf_eval_end.argtypes = [_P]
        L.trf_eval_gradient.restype = C.c_float
        L.trf_eval_gradient.argtypes = [_P, _P]
        L.trf_reset.argtypes = [_P]
        L.trf_update.argtypes = [_P]
        L.trf_set_lr.argtypes = [_P, C.c_float]
        L.trf_set_retrain.argtypes = [_P, C.c_int]
        L.lstm_eval.restype = _P
        L.lstm_eval.argtypes = [_P, C.c_int, _P]
        L.lstm_eval_end.argtypes = [_P]
        L.lstm_eval_gradient.restype = C.c_float
        L.lstm_eval_gradient.argtypes = [_P, _P]
        L.lstm_reset.argtypes = [_P]
        L.lstm_update.argtypes = [_P]
        L.nncp_process_block.argtypes = [_P, C.POINTER(NNCPPutBit), C.POINTER(NNCPGetBit), _P, C.c_int, C.c_int,
                                         C.c_int, C.POINTER(NNCPInterp), C.POINTER(NNCPStats)]
        L.nncp_retrain_block.argtypes = [_P, _P, C.c_int, C.POINTER(NNCPInterp), C.POINTER(NNCPStats)]
        L.nncp_fifo_symbol.argtypes = [_P, C.c_int, C.c_int, C.c_int]
        L.trf_last_logits.restype = _P
        L.nncp_model_last_logits.restype = _P
        L.nncp_model_last_logits.argtypes = [_P]
        L.trf_last_logits.argtypes = [_P]
        L.trf_step_begin.argtypes = [_P]
        L.trf_step_end.argtypes = [_P]
        L.trf_eval_step.restype = _P
        L.trf_eval_step.argtypes = [_P, C.c_int, _P]
        L.nncp_compress.restype = C.c_size_t
        L.nncp_compress.argtypes = [_P, _P, C.c_int, _P, C.c_size_t, C.c_int,
                                    C.POINTER(NNCPInterp), C.POINTER(NNCPStats)]
        L.nncp_decompress.argtypes = [_P, _P, C.c_size_t, _P, C.c_int, C.c_int,
                                      C.POINTER(NNCPInterp), C.POINTER(NNCPStats)]
        L.nncp_put_bit_init.argtypes = [C.POINTER(NNCPPutBit), _P, C.c_size_t]
        L.nncp_put_bit.argtypes = [C.POINTER(NNCPPutBit), C.c_int, C.c_int]
        L.nncp_put_bit_flush.restype = C.c_size_t
        L.nncp_put_bit_flush.argtypes = [C.POINTER(NNCPPutBit)]
        L.nncp_get_bit_init.argtypes = [C.POINTER(NNCPGetBit), _P, C.c_size_t]
        L.nncp_get_bit.argtypes = [C.POINTER(NNCPGetBit), C.c_int]
        L.nncp_write_sym.argtypes = [C.POINTER(NNCPPutBit), _P, C.c_int, C.c_int]
        L.nncp_read_sym.argtypes = [C.POINTER(NNCPGetBit), _P, C.c_int]
        L.nncp_write_sym_cdf.argtypes = [C.POINTER(NNCPPutBit), _P, C.c_int, C.c_int]
        L.nncp_read_sym_cdf.argtypes = [C.POINTER(NNCPGetBit), _P, C.c_int]
        L.nncp_write_sym_cdf_path.argtypes = [C.POINTER(NNCPPutBit), _P, C.c_int, C.c_int]
        L.nncp_interp.restype = C.c_float
        L.nncp_interp.argtypes = [C.POINTER(NNCPInterp), C.c_int64]
        L.nncp_profile.argtypes = [C.POINTER(NNCPConfig), C.POINTER(NNCPFileParams), C.c_char_p]
        L.nncp_parse_interp.argtypes = [C.POINTER(NNCPInterp), C.c_char_p]
        L.nncp_format_interp.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(NNCPInterp)]
        L.nncp_header_write.restype = C.c_size_t
        L.nncp_header_write.argtypes = [_P, C.c_size_t, C.POINTER(NNCPConfig), C.POINTER(NNCPFileParams)]
        L.nncp_header_read.argtypes = [_P, C.c_size_t, C.POINTER(NNCPConfig), C.POINTER(NNCPFileParams),
                                       C.POINTER(C.c_size_t)]
        L.nncp_block_len.argtypes = [C.POINTER(NNCPConfig), C.POINTER(NNCPInterp), C.c_int64, C.c_int64]
        L.nncp_encode_file.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(NNCPConfig), C.POINTER(NNCPFileParams),
                                       C.POINTER(NNCPStats), C.POINTER(NNCPStats)]
        L.nncp_decode_file.argtypes = [C.c_char_p, C.c_char_p, C.c_int, C.c_int, C.POINTER(NNCPStats),
                                       C.POINTER(NNCPStats)]
        L.nncp_put_bit_set_sink.argtypes = [C.POINTER(NNCPPutBit), _P, _P]
        # the libnc symbols the host library resolved (same handle namespace)
        self.ncl = C.CDLL(nc_libpath, mode=C.RTLD_LOCAL)
        # the tensor calls of the host code must land in that very library (and not in another
        # libnc that some earlier load put into the process-wide namespace)
        L.nncp_bound_libnc.restype = _P
        if L.nncp_bound_libnc() != C.cast(self.ncl.nc_context_init, _P).value:
            raise RuntimeError("%s is bound to another libnc than %s" % (libpath, nc_libpath))
        for name, (res, args) in B._PROTOS.items():
            f = getattr(self.ncl, name)
            f.restype, f.argtypes = res, args


def profile(host, name):
    """(NNCPConfig, NNCPFileParams) of one of nncp's profiles (nncp.c:2464-2636)."""
    cfg, fp = NNCPConfig(), NNCPFileParams()
    if host.lib.nncp_profile(C.byref(cfg), C.byref(fp), name.encode()) != 0:
        raise ValueError("unknown profile: %s" % name)
    return cfg, fp


def file_params(host, lr="3e-4", block_len="500000", use_bf16=0, max_size=-1, mode=0):
    fp = NNCPFileParams(use_bf16=use_bf16, max_size=max_size, mode=mode)
    for field, text in (("lr", lr), ("block_len", block_len)):
        if host.lib.nncp_parse_interp(C.byref(getattr(fp, field)), str(text).encode()) != 0:
            raise ValueError("bad schedule: %s" % text)
    return fp


def encode_file(host, src, dst, cfg, fp):
    """nncp c without the preprocessor; returns (coding stats, retrain stats)."""
    st, rst = NNCPStats(), NNCPStats()
    if host.lib.nncp_encode_file(os.fsencode(src), os.fsencode(dst), C.byref(cfg), C.byref(fp),
                                 C.byref(st), C.byref(rst)) != 0:
        raise RuntimeError("encoding %s failed" % src)
    return st, rst


def decode_file(host, src, dst, use_device=1, nb_threads=1):
    st, rst = NNCPStats(), NNCPStats()
    if host.lib.nncp_decode_file(os.fsencode(src), os.fsencode(dst), use_device, nb_threads,
                                 C.byref(st), C.byref(rst)) != 0:
        raise RuntimeError("decoding %s failed" % src)
    return st, rst


class Model:
    """One NNCPModel plus helpers to move numpy data in and out."""

    def __init__(self, host, cfg):
        self.host, self.cfg, self.L, self.nc = host, cfg, host.lib, host.ncl
        self.ptr = self.L.nncp_model_new(C.byref(cfg))
        self.dev = self.L.nncp_model_device(self.ptr)
        self.cpu = self.L.nncp_model_cpu_device(self.ptr)
        self.ctx = self.L.nncp_model_context(self.ptr)
        # the entry points of the model class in use (trf_* or lstm_*)
        pre = "lstm" if cfg.model_type == MODEL_LSTM else "trf"
        self._eval, self._eval_end = getattr(self.L, pre + "_eval"), getattr(self.L, pre + "_eval_end")
        self._eval_gradient, self._update = getattr(self.L, pre + "_eval_gradient"), getattr(self.L, pre + "_update")
        self._reset = getattr(self.L, pre + "_reset")

    def close(self):
        if self.ptr:
            self.L.nncp_model_free(self.ptr)
            self.ptr = None

    # -- tensors ---------------------------------------------------------
    def _to_numpy(self, x):
        d = (C.c_size_t * 8)()
        n = self.nc.nc_tensor_get_dims(x, d)
        dims = tuple(d[i] for i in range(n))
        t = self.nc.nc_tensor_get_item_type(x)
        h = self.nc.nc_tensor_to_cpu_device(self.nc.nc_dup_tensor(x))
        cnt = int(np.prod(dims)) if dims else 1
        ptr = self.nc.nc_tensor_get_ptr(h, None)
        dt = np.dtype(B._NP[t])
        buf = (C.c_char * (cnt * dt.itemsize)).from_address(ptr)
        out = np.frombuffer(buf, dtype=dt).copy().reshape(tuple(reversed(dims)))
        if t == B.BF16:
            out = B.bf16_widen(out)
        self.nc.nc_free_tensor(h)
        return out

    def _host_tensor(self, arr):
        arr = np.ascontiguousarray(arr) if np.ndim(arr) else np.asarray(arr)
        dims = (C.c_size_t * max(arr.ndim, 1))(*reversed(arr.shape))
        x = self.nc.nc_new_tensor_nz(self.cpu, B._NC[arr.dtype], arr.ndim, dims)
        C.memmove(self.nc.nc_tensor_get_ptr(x, None), arr.ctypes.data, arr.nbytes)
        return x

    def _symbols(self, a):
        """Token ids as int32, refused when one lies outside the alphabet: on the device they
        index the embedding table and the probability columns unchecked."""
        a = np.asarray(a, dtype=np.int32)
        if a.size and (a.min() < 0 or a.max() >= self.cfg.n_symbols):
            raise ValueError("symbol outside [0, %d)" % self.cfg.n_symbols)
        return a

    def param_names(self):
        n = self.L.nncp_model_param_count(self.ptr)
        return [self.L.nncp_model_param_name(self.ptr, i).decode() for i in range(n)]

    def get_param(self, name):
        return self._to_numpy(self.L.nncp_model_param(self.ptr, name.encode())[0])

    def set_param(self, name, arr):
        slot = self.L.nncp_model_param(self.ptr, name.encode())
        arr = np.asarray(arr, dtype=np.float32)
        if self.nc.nc_tensor_get_item_type(slot[0]) == B.BF16:     # a bf16 parameter takes the rounding
            dims = (C.c_size_t * max(arr.ndim, 1))(*reversed(arr.shape))
            h = self.nc.nc_new_tensor_nz(self.cpu, B.BF16, arr.ndim, dims)
            bits = np.ascontiguousarray(B.bf16_bits(arr))
            C.memmove(self.nc.nc_tensor_get_ptr(h, None), bits.ctypes.data, bits.nbytes)
        else:
            h = self._host_tensor(arr)
        src = self.nc.nc_tensor_to_device(h, self.dev)
        self.nc.nc_tensor_copy(slot[0], src)
        self.nc.nc_free_tensor(src)

    def params(self):
        return {n: self.get_param(n) for n in self.param_names()}

    def state(self):
        """Everything one training step hands to the next: parameters, the optimiser's second
        moments and the per-layer memories, as numpy arrays (a checkpoint)."""
        names = self.param_names()
        v = {}
        for n in names:
            t = self.L.nncp_model_opt_state(self.ptr, n.encode(), 1)
            if t:
                v[n] = self._to_numpy(t)
                self.nc.nc_free_tensor(t)
        mem = []
        for l in range(self.cfg.n_layer):
            t = self.L.nncp_model_memory(self.ptr, l)
            if t:
                mem.append(self._to_numpy(t))
        return dict(w={n: self.get_param(n) for n in names}, v=v, mem=mem)

    def load_state(self, st):
        """Puts the model into a state taken from another model of the same configuration,
        on either library (see state())."""
        for n, a in st["w"].items():
            self.set_param(n, a)
        for n, a in st["v"].items():
            h = self._host_tensor(np.ascontiguousarray(a, dtype=np.float32).ravel())
            self.L.nncp_model_set_opt_state(self.ptr, n.encode(), 1, h)
            self.nc.nc_free_tensor(h)
        for l, a in enumerate(st["mem"]):
            dst = self.L.nncp_model_memory(self.ptr, l)
            src = self.nc.nc_tensor_to_device(self._host_tensor(np.ascontiguousarray(a, dtype=np.float32)), self.dev)
            self.nc.nc_tensor_copy(dst, src)
            self.nc.nc_free_tensor(src)

    def save_coefs(self, path):
        """Every parameter to a parameter file (nc_save_coefs, libnc.h:530)."""
        self.L.nncp_model_save_coefs(self.ptr, os.fsencode(path))

    def load_coefs(self, path):
        """Parameters from a file written by save_coefs of a model of the same
        configuration, on either library (nc_load_coefs, libnc.h:536)."""
        self.L.nncp_model_load_coefs(self.ptr, os.fsencode(path))

    # -- the model class ---------------------------------------------------
    def eval(self, tokens, output_index=-1, keep=False):
        """tokens: int array (T, B) [numpy order of the (B, T) input tensor].
        Returns the probabilities as numpy (T|1, B, V)."""
        inp = self._host_tensor(self._symbols(tokens))
        out = self._eval(self.ptr, output_index, inp)
        self.nc.nc_free_tensor(inp)
        res = self._to_numpy(out)
        self.nc.nc_free_tensor(out)
        if not keep:
            self._eval_end(self.ptr)
        return res

    def logits(self):
        return self._to_numpy(self.L.nncp_model_last_logits(self.ptr))

    def eval_steps(self, tokens):
        """Per-timestep cached evaluation of a whole segment (trf_step_begin +
        trf_eval_step for every position).  Returns (probabilities (T, B, V),
        logits (T, B, V)) assembled from the single-column results."""
        tokens = self._symbols(tokens)
        inp = self._host_tensor(tokens)
        self.L.trf_step_begin(self.ptr)
        probs, logits = [], []
        for t in range(tokens.shape[0]):
            out = self.L.trf_eval_step(self.ptr, t, inp)
            probs.append(self._to_numpy(out)[0])
            logits.append(self.logits()[0])
            self.nc.nc_free_tensor(out)
        self.L.trf_step_end(self.ptr)
        self.nc.nc_free_tensor(inp)
        return np.stack(probs), np.stack(logits)

    def train_step(self, tokens, targets, lr):
        """One full-segment evaluation + gradient + update; returns
        (probabilities, loss in nats summed over the segment)."""
        p = self.eval(tokens, -1, keep=True)
        tgt = self._host_tensor(self._symbols(targets))
        self.L.trf_set_lr(self.ptr, lr)  # both classes: nc_sgd_opt_set_lr on the model's optimiser
        loss = self._eval_gradient(self.ptr, tgt)
        self.nc.nc_free_tensor(tgt)
        self._update(self.ptr)
        return p, -loss

    def compress(self, syms, mode, lr=3e-4):
        syms = np.ascontiguousarray(syms, dtype=np.uint16)
        cap = syms.size * 4 + 1024
        out = np.zeros(cap, dtype=np.uint8)
        st = NNCPStats()
        sched = constant_lr(lr) if not isinstance(lr, NNCPInterp) else lr
        n = self.L.nncp_compress(self.ptr, syms.ctypes.data, syms.size, out.ctypes.data, cap, mode,
                                 C.byref(sched), C.byref(st))
        return out[:n].copy(), st

    def decompress(self, data, n_syms, mode, lr=3e-4):
        data = np.ascontiguousarray(data, dtype=np.uint8)
        out = np.zeros(n_syms, dtype=np.uint16)
        st = NNCPStats()
        sched = constant_lr(lr) if not isinstance(lr, NNCPInterp) else lr
        self.L.nncp_decompress(self.ptr, data.ctypes.data, data.size, out.ctypes.data, n_syms, mode,
                               C.byref(sched), C.byref(st))
        return out, st

    # -- several blocks through one coder, with the retrain pass between them ----
    def compress_blocks(self, syms, block_len, mode, lr=3e-4):
        """The reference's file loop (nncp.c:3375-3460, in memory): blocks of
        block_len symbols through ONE range coder, nncp_retrain_block after
        each.  Returns (bytes, coding stats, retrain stats)."""
        syms = np.ascontiguousarray(syms, dtype=np.uint16)
        cap = syms.size * 4 + 1024
        out = np.zeros(cap, dtype=np.uint8)
        st, rst = NNCPStats(), NNCPStats()
        sched = constant_lr(lr) if not isinstance(lr, NNCPInterp) else lr
        pb = NNCPPutBit()
        self.L.nncp_put_bit_init(C.byref(pb), out.ctypes.data, cap)
        for pos in range(0, syms.size, block_len):
            blk = syms[pos:pos + block_len].copy()
            self.L.nncp_process_block(self.ptr, C.byref(pb), None, blk.ctypes.data, blk.size, 0, mode,
                                      C.byref(sched), C.byref(st))
            self.L.nncp_retrain_block(self.ptr, blk.ctypes.data, blk.size, C.byref(sched), C.byref(rst))
        n = self.L.nncp_put_bit_flush(C.byref(pb))
        if pb.overflow:
            raise RuntimeError("output buffer too small")
        return out[:n].copy(), st, rst

    def decompress_blocks(self, data, n_syms, block_len, mode, lr=3e-4):
        data = np.ascontiguousarray(data, dtype=np.uint8)
        out = np.zeros(n_syms, dtype=np.uint16)
        st, rst = NNCPStats(), NNCPStats()
        sched = constant_lr(lr) if not isinstance(lr, NNCPInterp) else lr
        gb = NNCPGetBit()
        self.L.nncp_get_bit_init(C.byref(gb), data.ctypes.data, data.size)
        for pos in range(0, n_syms, block_len):
            blk = out[pos:pos + block_len]
            self.L.nncp_process_block(self.ptr, None, C.byref(gb), blk.ctypes.data, blk.size, 1, mode,
                                      C.byref(sched), C.byref(st))
            self.L.nncp_retrain_block(self.ptr, blk.ctypes.data, blk.size, C.byref(sched), C.byref(rst))
        return out, st, rst
