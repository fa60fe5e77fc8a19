"""ctypes binding of include/coalsack_moe.h.

Loads the in-tree ``libcoalsack_moe.so`` and fails loudly when it is missing:
there is no fallback path of any kind.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

OK, ERR_ARG, ERR_HIP, ERR_RANGE, ERR_ALL_EMPTY, ERR_SCALE, ERR_STATE = range(7)
ACT_MODIFIED_SWIGLU, ACT_STANDARD_SWIGLU = 0, 1
W_UP, W_GATE, W_DOWN = 0, 1, 2
FWD_RMSNORM, FWD_RESIDUAL = 1, 2

# name -> (restype, argtypes); every symbol include/coalsack_moe.h declares
_P = C.c_void_p
_F = C.POINTER(C.c_float)
_B = C.POINTER(C.c_uint8)
_I64 = C.c_int64
SIGNATURES = {
    "csk_init": (C.c_int, [C.c_int]),
    "csk_last_error": (C.c_char_p, []),
    "csk_device_info": (C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_size_t)]),
    "csk_device_memory": (C.c_int, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "csk_alloc_count": (C.c_int, [C.POINTER(C.c_uint64)]),
    "csk_dev_alloc": (_P, [C.c_size_t]),
    "csk_dev_free": (None, [_P]),
    "csk_copy_h2d": (C.c_int, [_P, _P, C.c_size_t]),
    "csk_copy_d2h": (C.c_int, [_P, _P, C.c_size_t]),
    "csk_copy_d2d": (C.c_int, [_P, _P, C.c_size_t]),
    "csk_synchronize": (C.c_int, []),
    "csk_event_create": (_P, []),
    "csk_event_destroy": (None, [_P]),
    "csk_event_record": (C.c_int, [_P]),
    "csk_event_elapsed_ms": (C.c_int, [_P, _P, _F]),
    "csk_stage_timing": (C.c_int, [C.c_int]),
    "csk_stage_times": (C.c_int, [_F]),
    "csk_kernel_times": (C.c_int, [_F]),
    "csk_mxfp4_upload": (C.c_int, [_P, _I64, _I64, C.POINTER(_P)]),
    "csk_mxfp4_free": (None, [_P]),
    "csk_mxfp4_dequant": (C.c_int, [_P, _P]),
    "csk_mxfp4_export": (C.c_int, [_P, _P]),
    "csk_f16_upload": (C.c_int, [_P, _I64, _I64, C.POINTER(_P)]),
    "csk_f16_upload_ggml": (C.c_int, [C.c_int, _P, _I64, _I64, C.POINTER(_P)]),
    "csk_f16_upload_f32": (C.c_int, [_P, _I64, _I64, C.POINTER(_P)]),
    "csk_f16_free": (None, [_P]),
    "csk_f16_export": (C.c_int, [_P, _P]),
    "csk_layer_create": (C.c_int, [_I64, _I64, _I64, _I64, C.POINTER(_P)]),
    "csk_layer_create_f16": (C.c_int, [_I64, _I64, _I64, _I64, C.POINTER(_P)]),
    "csk_layer_set_expert_f16": (C.c_int, [_P, _I64, _P, _P, _P, _P, _P, _P]),
    "csk_layer_set_expert_matrix": (C.c_int, [_P, _I64, C.c_int, C.c_int, _P]),
    "csk_layer_export_f16": (C.c_int, [_P, _I64, C.c_int, _P]),
    "csk_layer_destroy": (None, [_P]),
    "csk_layer_set_options": (C.c_int, [_P, C.c_int, C.c_int, C.c_int]),
    "csk_layer_set_router": (C.c_int, [_P, _P, _P]),
    "csk_layer_set_expert": (C.c_int, [_P, _I64, _P, _P, _P, _P, _P, _P]),
    "csk_layer_set_norm": (C.c_int, [_P, _P, C.c_float]),
    "csk_layer_fill_synthetic": (C.c_int, [_P, C.c_uint64, _I64, C.c_int, C.c_int]),
    "csk_layer_dequant": (C.c_int, [_P, _I64, C.c_int, _P]),
    "csk_layer_export": (C.c_int, [_P, _I64, C.c_int, _P]),
    "csk_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(_P)]),
    "csk_gguf_open_shards": (C.c_int, [C.POINTER(C.c_char_p), _I64, C.POINTER(_P)]),
    "csk_gguf_tensor_shard": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_int32)]),
    "csk_gguf_close": (None, [_P]),
    "csk_gguf_tensor_count": (C.c_int, [_P, C.POINTER(_I64)]),
    "csk_gguf_tensor_name": (C.c_int, [_P, _I64, C.c_char_p, C.c_size_t]),
    "csk_gguf_tensor_info": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_int32),
                                        C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                        C.POINTER(C.c_uint64)]),
    "csk_gguf_get_u32": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_uint32)]),
    "csk_gguf_get_str": (C.c_int, [_P, C.c_char_p, C.c_char_p, C.c_size_t]),
    "csk_layer_from_gguf": (C.c_int, [_P, _I64, C.POINTER(_P)]),
    "csk_moe_forward": (C.c_int, [_P, _P, _I64, _P, C.c_int]),
    "csk_moe_forward_noalloc": (C.c_int, [_P, _P, _I64, _P, C.c_int]),
    "csk_moe_forward_host": (C.c_int, [_P, _P, _I64, _P, _P, C.c_int]),
    "csk_moe_stack_forward": (C.c_int, [C.POINTER(_P), _I64, _P, _I64]),
    "csk_set_pass_tokens": (C.c_int, [_I64]),
    "csk_layer_last_dispatch": (C.c_int, [_P, _P, _P]),
    "csk_moe_router": (C.c_int, [_P, _I64, _I64, _P, _I64, _P, _I64, C.c_int, _P]),
    "csk_moe_router_resident": (C.c_int, [_P, _I64, _I64, _P, _I64, _P, _I64, C.c_int, _P]),
    "csk_moe_router_logits": (C.c_int, [_P, _I64, _I64, _P, _I64, _P, _P]),
    "csk_expert_mlp_mxfp4": (C.c_int, [C.c_int, _P, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P,
                                       _I64, C.c_int, C.c_int, _P, C.POINTER(C.c_int)]),
    "csk_expert_mlp_f16": (C.c_int, [C.c_int, _P, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P,
                                     _I64, C.c_int, C.c_int, _P, C.POINTER(C.c_int)]),
    "csk_dense_ffn_f16": (C.c_int, [_P, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "csk_matmul_transpose_f16": (C.c_int, [_P, _I64, _I64, _P, _P]),
    "csk_expert_token_mxfp4": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, C.c_int]),
    "csk_expert_merge": (C.c_int, [_P, _I64, _I64, _I64, _I64, C.POINTER(_P), C.c_int, _P]),
    "csk_rmsnorm": (C.c_int, [_P, _P, _P, _I64, _I64, C.c_float]),
    "csk_rmsnorm_f64": (C.c_int, [_P, _P, _P, _I64, _I64, C.c_float]),
    "csk_add": (C.c_int, [_P, _P, _P, _I64]),
    "csk_add_broadcast": (C.c_int, [_P, _P, C.c_int, _P, _P, C.c_int, C.c_int, _P]),
    "csk_moe_router_f64": (C.c_int, [_P, _I64, _I64, _P, _I64, _P, _I64, C.c_int, _P, _P]),
    "csk_layer_create_view": (C.c_int, [_I64, _I64, _I64, _I64, C.POINTER(_P)]),
    "csk_layer_attach_expert": (C.c_int, [_P, _I64, _P, _P, _P, _P, _P, _P]),
    "csk_layer_detach_expert": (C.c_int, [_P, _I64]),
    "csk_moe_frame_begin": (C.c_int, [_P, _P, _I64, _P, C.c_int, C.POINTER(C.c_int)]),
    "csk_moe_frame_expert_rows": (C.c_int, [_P, _I64, _P]),
    "csk_moe_frame_void": (C.c_int, [_P]),
    "csk_moe_frame_merged": (C.c_int, [_P, _P, C.POINTER(C.c_int)]),
}


class CskError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"[csk error {code}] {message}")
        self.code = code
        self.message = message


def lib_path():
    """The in-tree library, or the file COALSACK_MOE_LIB names (another build of it)."""
    return os.environ.get("COALSACK_MOE_LIB") or os.path.join(_HERE, "libcoalsack_moe.so")


def _ptr(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "array must be contiguous"
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.uint8)


class Library:
    """Thin object wrapper; every method maps to one C entry point."""

    def __init__(self, path=None):
        path = path or lib_path()
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        self.dll = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.dll, name)  # AttributeError if a declared symbol is not exported
            fn.restype = res
            fn.argtypes = args
        self.initialised = False

    # -- helpers
    def check(self, rc):
        if rc != OK:
            raise CskError(rc, self.dll.csk_last_error().decode(errors="replace"))

    def init(self, device=0):
        self.check(self.dll.csk_init(device))
        self.initialised = True
        return self

    def device_info(self):
        name = C.create_string_buffer(256)
        cus = C.c_int()
        mem = C.c_size_t()
        self.check(self.dll.csk_device_info(name, 256, C.byref(cus), C.byref(mem)))
        return name.value.decode(), cus.value, mem.value

    def device_memory(self):
        """(free, total) bytes of device memory as the runtime reports them now."""
        free, total = C.c_size_t(), C.c_size_t()
        self.check(self.dll.csk_device_memory(C.byref(free), C.byref(total)))
        return free.value, total.value

    def alloc_count(self):
        """Device allocations the library has made in this process so far."""
        n = C.c_uint64()
        self.check(self.dll.csk_alloc_count(C.byref(n)))
        return n.value

    # -- device memory
    def dev_alloc(self, nbytes):
        p = self.dll.csk_dev_alloc(nbytes)
        if not p:
            raise CskError(ERR_HIP, self.dll.csk_last_error().decode(errors="replace"))
        return p

    def dev_free(self, p):
        self.dll.csk_dev_free(p)

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.dev_alloc(arr.nbytes)
        self.check(self.dll.csk_copy_h2d(p, _ptr(arr), arr.nbytes))
        return p

    def to_host(self, p, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self.check(self.dll.csk_copy_d2h(_ptr(out), p, out.nbytes))
        return out

    def copy_d2d(self, dst, src, nbytes):
        self.check(self.dll.csk_copy_d2d(dst, src, nbytes))

    def set_pass_tokens(self, tokens):
        self.check(self.dll.csk_set_pass_tokens(tokens))

    def synchronize(self):
        self.check(self.dll.csk_synchronize())

    def event(self):
        e = self.dll.csk_event_create()
        if not e:
            raise CskError(ERR_HIP, "csk_event_create failed")
        return e

    def record(self, e):
        self.check(self.dll.csk_event_record(e))

    def elapsed_ms(self, a, b):
        ms = C.c_float()
        self.check(self.dll.csk_event_elapsed_ms(a, b, C.byref(ms)))
        return ms.value

    STAGES = ("prep", "router", "dispatch", "gateup", "down", "combine")

    def stage_timing(self, on):
        self.check(self.dll.csk_stage_timing(int(on)))

    def stage_times(self):
        ms = (C.c_float * len(self.STAGES))()
        self.check(self.dll.csk_stage_times(ms))
        return dict(zip(self.STAGES, list(ms)))

    def kernel_times(self):
        """(gate/up, down) kernel durations in ms of the last forward under stage timing."""
        ms = (C.c_float * 2)()
        self.check(self.dll.csk_kernel_times(ms))
        return ms[0], ms[1]

    # -- MXFP4 matrices
    def mxfp4_upload(self, blocks, rows, K):
        blocks = _u8(blocks)
        assert blocks.size == rows * (K // 32) * 17
        h = _P()
        self.check(self.dll.csk_mxfp4_upload(_ptr(blocks), rows, K, C.byref(h)))
        return h

    def mxfp4_free(self, h):
        self.dll.csk_mxfp4_free(h)

    def mxfp4_dequant(self, h, rows, K):
        out = np.empty((rows, K), np.float32)
        self.check(self.dll.csk_mxfp4_dequant(h, _ptr(out)))
        return out

    def mxfp4_export(self, h, rows, K):
        out = np.empty(rows * (K // 32) * 17, np.uint8)
        self.check(self.dll.csk_mxfp4_export(h, _ptr(out)))
        return out

    # -- fp16 matrices
    def f16_upload(self, w):
        """w: float16 [rows, K], row-major."""
        w = np.ascontiguousarray(w, dtype=np.float16)
        rows, K = w.shape
        h = _P()
        self.check(self.dll.csk_f16_upload(_ptr(w), rows, K, C.byref(h)))
        return h

    def f16_upload_f32(self, w):
        """fp32 [rows, K] weights kept as two fp16 terms (csk_f16_upload_f32)."""
        w = _f32(w)
        h = _P()
        self.check(self.dll.csk_f16_upload_f32(_ptr(w), w.shape[0], w.shape[1], C.byref(h)))
        return h

    def f16_upload_ggml(self, ggml_type, data, rows, K):
        """data: uint8 stream of a [rows, K] matrix stored as ggml F16 (1), Q4_K (12) or Q6_K (14)."""
        data = _u8(data)
        h = _P()
        self.check(self.dll.csk_f16_upload_ggml(ggml_type, _ptr(data), rows, K, C.byref(h)))
        return h

    def f16_free(self, h):
        self.dll.csk_f16_free(h)

    def f16_export(self, h, rows, K):
        out = np.empty((rows, K), np.float16)
        self.check(self.dll.csk_f16_export(h, _ptr(out)))
        return out

    def expert_mlp_f16(self, expert_id, hidden, w_up, w_gate, w_down, b_up, b_gate, b_down, pairs,
                       act=ACT_MODIFIED_SWIGLU, weight_before_ffn=False):
        """w_*: float16 arrays [F,H], [F,H], [H,F]; uploads them, runs the node, frees them."""
        hidden, pairs = _f32(hidden), _f32(pairs)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        T, H = hidden.shape
        F = w_up.shape[0]
        k = pairs.shape[1]
        hs = [self.f16_upload(w) for w in (w_up, w_gate, w_down)]
        try:
            out = np.empty((T, H), np.float32)
            empty = C.c_int()
            self.check(self.dll.csk_expert_mlp_f16(
                expert_id, _ptr(hidden), T, H, F, hs[0], hs[1], hs[2], _ptr(b_up), _ptr(b_gate),
                _ptr(b_down), _ptr(pairs), k, act, int(weight_before_ffn), _ptr(out),
                C.byref(empty)))
        finally:
            for h in hs:
                self.f16_free(h)
        return None if empty.value else out

    def dense_ffn_f16(self, hidden, w_gate, w_up, w_down, b_gate=None, b_up=None, b_down=None):
        """dense_ffn_node with float16 (or float32) weights [F,H], [F,H], [H,F]; uploads them for the call."""
        hidden = _f32(hidden)
        b_gate, b_up, b_down = _f32(b_gate), _f32(b_up), _f32(b_down)
        T, H = hidden.shape
        F = w_gate.shape[0]
        up = self.f16_upload_f32 if w_gate.dtype == np.float32 else self.f16_upload
        hs = [up(w) for w in (w_gate, w_up, w_down)]
        try:
            out = np.empty((T, H), np.float32)
            self.check(self.dll.csk_dense_ffn_f16(_ptr(hidden), T, H, F, hs[0], hs[1], hs[2], _ptr(b_gate),
                                                  _ptr(b_up), _ptr(b_down), _ptr(out)))
        finally:
            for h in hs:
                self.f16_free(h)
        return out

    def matmul_transpose_f16(self, a, w):
        """a [M,K] f32 x w [N,K]^T (float16 or float32) -> [M,N]; uploads w for the call."""
        a = _f32(a)
        M, K = a.shape
        h = self.f16_upload_f32(w) if w.dtype == np.float32 else self.f16_upload(w)
        try:
            out = np.empty((M, w.shape[0]), np.float32)
            self.check(self.dll.csk_matmul_transpose_f16(_ptr(a), M, K, h, _ptr(out)))
        finally:
            self.f16_free(h)
        return out

    # -- node-level ops
    def moe_router(self, hidden, gate_w, gate_b, k, sigmoid=False):
        hidden, gate_w, gate_b = _f32(hidden), _f32(gate_w), _f32(gate_b)
        T, H = hidden.shape
        E = gate_w.shape[0]
        out = np.empty((T, k, 2), np.float32)
        self.check(self.dll.csk_moe_router(_ptr(hidden), T, H, _ptr(gate_w), E, _ptr(gate_b), k,
                                           int(sigmoid), _ptr(out)))
        return out

    def moe_router_resident(self, hidden, gate_w_dev, E, gate_b_dev, k, sigmoid=False):
        """csk_moe_router with the gate [E,H] (and bias, or None) already in device memory."""
        hidden = _f32(hidden)
        T, H = hidden.shape
        out = np.empty((T, k, 2), np.float32)
        self.check(self.dll.csk_moe_router_resident(_ptr(hidden), T, H, C.c_void_p(gate_w_dev), E,
                                                    C.c_void_p(gate_b_dev) if gate_b_dev else None, k,
                                                    int(sigmoid), _ptr(out)))
        return out

    def moe_router_f64(self, hidden, gate_w, gate_b, k, sigmoid=False, want_logits=False):
        """moe_router_node on float64 inputs: float32 pairs [T,k,2] (and the float64 logits)."""
        hidden = np.ascontiguousarray(hidden, np.float64)
        gate_w = np.ascontiguousarray(gate_w, np.float64)
        gate_b = _f32(gate_b)
        T, H = hidden.shape
        E = gate_w.shape[0]
        out = np.empty((T, k, 2), np.float32)
        logits = np.empty((T, E), np.float64) if want_logits else None
        self.check(self.dll.csk_moe_router_f64(_ptr(hidden), T, H, _ptr(gate_w), E, _ptr(gate_b), k,
                                               int(sigmoid), _ptr(out), _ptr(logits)))
        return (out, logits) if want_logits else out

    ADD_DTYPES = {np.dtype(np.float32): 0, np.dtype(np.float64): 1, np.dtype(np.int32): 2, np.dtype(np.int64): 3}

    def add_broadcast(self, a, b):
        """add_node with broadcasting; both arrays float32, float64, int32 or int64."""
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        if a.dtype != b.dtype:
            raise ValueError("add: input dtype mismatch")
        sa, sb = np.array(a.shape, np.int64), np.array(b.shape, np.int64)
        try:
            shape = np.broadcast_shapes(a.shape, b.shape)
        except ValueError:
            shape = (0,)
        out = np.empty(shape, a.dtype)
        self.check(self.dll.csk_add_broadcast(_ptr(a), _ptr(sa), a.ndim, _ptr(b), _ptr(sb), b.ndim,
                                              self.ADD_DTYPES[a.dtype], _ptr(out)))
        return out

    def moe_router_logits(self, hidden, gate_w, gate_b):
        hidden, gate_w = _f32(hidden), _f32(gate_w)
        T, H = hidden.shape
        E = gate_w.shape[0]
        gb = _f32(gate_b) if gate_b is not None else None
        out = np.empty((T, E), np.float32)
        self.check(self.dll.csk_moe_router_logits(_ptr(hidden), T, H, _ptr(gate_w), E,
                                                  _ptr(gb) if gb is not None else None, _ptr(out)))
        return out

    def expert_mlp(self, expert_id, hidden, F, h_up, h_gate, h_down, b_up, b_gate, b_down, pairs,
                   act=ACT_MODIFIED_SWIGLU, weight_before_ffn=False):
        hidden, pairs = _f32(hidden), _f32(pairs)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        T, H = hidden.shape
        k = pairs.shape[1]
        out = np.empty((T, H), np.float32)
        empty = C.c_int()
        self.check(self.dll.csk_expert_mlp_mxfp4(
            expert_id, _ptr(hidden), T, H, F, h_up, h_gate, h_down, _ptr(b_up), _ptr(b_gate),
            _ptr(b_down), _ptr(pairs), k, act, int(weight_before_ffn), _ptr(out), C.byref(empty)))
        return None if empty.value else out

    def expert_token(self, x, w_up, w_gate, w_down, b_up, b_gate, b_down, H, F,
                     act=ACT_MODIFIED_SWIGLU):
        x, w_up, w_gate, w_down = _f32(x), _u8(w_up), _u8(w_gate), _u8(w_down)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        out = np.empty(H, np.float32)
        self.check(self.dll.csk_expert_token_mxfp4(_ptr(x), _ptr(w_up), _ptr(w_gate), _ptr(w_down),
                                                   _ptr(b_up), _ptr(b_gate), _ptr(b_down),
                                                   _ptr(out), H, F, act))
        return out

    def expert_merge(self, pairs, expert_outs, H, pre_weighted=False):
        pairs = _f32(pairs)
        T, k = pairs.shape[:2]
        E = len(expert_outs)
        keep = [_f32(a) for a in expert_outs]
        arr = (_P * E)(*[(_ptr(a) if a is not None else None) for a in keep])
        out = np.empty((T, H), np.float32)
        self.check(self.dll.csk_expert_merge(_ptr(pairs), T, k, E, H, arr, int(pre_weighted),
                                             _ptr(out)))
        return out

    def rmsnorm(self, x, w, eps):
        x, w = _f32(x), _f32(w)
        T, H = x.shape
        out = np.empty((T, H), np.float32)
        self.check(self.dll.csk_rmsnorm(_ptr(x), _ptr(w), _ptr(out), T, H, eps))
        return out

    def rmsnorm_f64(self, x, w, eps):
        x = np.ascontiguousarray(x, np.float64)
        w = np.ascontiguousarray(w, np.float64)
        T, H = x.shape
        out = np.empty((T, H), np.float64)
        self.check(self.dll.csk_rmsnorm_f64(_ptr(x), _ptr(w), _ptr(out), T, H, eps))
        return out

    def add(self, a, b):
        a, b = _f32(a), _f32(b)
        out = np.empty(a.shape, np.float32)
        self.check(self.dll.csk_add(_ptr(a), _ptr(b), _ptr(out), a.size))
        return out

    # -- layer
    def layer(self, E, k, H, F, f16=False):
        return Layer(self, E, k, H, F, f16=f16)

    def gguf(self, path):
        return Gguf(self, path)


class Gguf:
    """An open GGUF checkpoint (csk_gguf_*): metadata and tensor table, no GPU needed.
    `path` is one file, or the list of shard files of a split checkpoint."""

    def __init__(self, lib, path):
        self.lib = lib
        self.h = _P()
        if isinstance(path, (list, tuple)):
            arr = (C.c_char_p * len(path))(*[os.fsencode(p) for p in path])
            lib.check(lib.dll.csk_gguf_open_shards(arr, len(path), C.byref(self.h)))
        else:
            lib.check(lib.dll.csk_gguf_open(os.fsencode(path), C.byref(self.h)))

    def close(self):
        if self.h:
            self.lib.dll.csk_gguf_close(self.h)
            self.h = _P()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def tensor_names(self):
        n = _I64()
        self.lib.check(self.lib.dll.csk_gguf_tensor_count(self.h, C.byref(n)))
        buf = C.create_string_buffer(512)
        out = []
        for i in range(n.value):
            self.lib.check(self.lib.dll.csk_gguf_tensor_name(self.h, i, buf, 512))
            out.append(buf.value.decode(errors="replace"))
        return out

    def tensor_info(self, name):
        t, nd, off, nb = C.c_uint32(), C.c_int32(), C.c_uint64(), C.c_uint64()
        dims = (C.c_uint64 * 4)()
        self.lib.check(self.lib.dll.csk_gguf_tensor_info(self.h, name.encode(), C.byref(t), C.byref(nd),
                                                         dims, C.byref(off), C.byref(nb)))
        return dict(type=t.value, dims=list(dims)[:nd.value], offset=off.value, nbytes=nb.value)

    def tensor_shard(self, name):
        sh = C.c_int32()
        self.lib.check(self.lib.dll.csk_gguf_tensor_shard(self.h, name.encode(), C.byref(sh)))
        return sh.value

    def get_u32(self, key):
        v = C.c_uint32()
        self.lib.check(self.lib.dll.csk_gguf_get_u32(self.h, key.encode(), C.byref(v)))
        return v.value

    def get_str(self, key):
        buf = C.create_string_buffer(1024)
        self.lib.check(self.lib.dll.csk_gguf_get_str(self.h, key.encode(), buf, 1024))
        return buf.value.decode(errors="replace")

    def layer(self, block):
        """Resident MoE layer of transformer block `block` (csk_layer_from_gguf)."""
        h = _P()
        self.lib.check(self.lib.dll.csk_layer_from_gguf(self.h, block, C.byref(h)))
        arch = self.get_str("general.architecture")
        gi = self.tensor_info(f"blk.{block}.ffn_gate_inp.weight")
        up = self.tensor_info(f"blk.{block}.ffn_up_exps.weight")
        return Layer.adopt(self.lib, h, gi["dims"][1], self.get_u32(arch + ".expert_used_count"),
                           gi["dims"][0], up["dims"][1], f16=up["type"] != 39)


class Layer:
    """One resident MoE layer (csk_layer_*)."""

    def __init__(self, lib, E, k, H, F, f16=False):
        self.lib, self.E, self.k, self.H, self.F, self.f16 = lib, E, k, H, F, f16
        self.h = _P()
        create = lib.dll.csk_layer_create_f16 if f16 else lib.dll.csk_layer_create
        lib.check(create(E, k, H, F, C.byref(self.h)))

    @classmethod
    def adopt(cls, lib, handle, E, k, H, F, f16=False):
        """Wraps a layer handle the library created itself."""
        self = cls.__new__(cls)
        self.lib, self.E, self.k, self.H, self.F, self.h, self.f16 = lib, E, k, H, F, handle, f16
        return self

    def close(self):
        if self.h:
            self.lib.dll.csk_layer_destroy(self.h)
            self.h = _P()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def set_options(self, sigmoid=False, act=ACT_MODIFIED_SWIGLU, weight_before_ffn=False):
        self.lib.check(self.lib.dll.csk_layer_set_options(self.h, int(sigmoid), act,
                                                          int(weight_before_ffn)))

    def set_router(self, gate_w, gate_b=None):
        gate_w, gate_b = _f32(gate_w), _f32(gate_b)
        assert gate_w.shape == (self.E, self.H)
        self.lib.check(self.lib.dll.csk_layer_set_router(self.h, _ptr(gate_w), _ptr(gate_b)))

    def set_expert(self, e, w_up, w_gate, w_down, b_up=None, b_gate=None, b_down=None):
        w_up, w_gate, w_down = _u8(w_up), _u8(w_gate), _u8(w_down)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        self.lib.check(self.lib.dll.csk_layer_set_expert(
            self.h, e, _ptr(w_up), _ptr(w_gate), _ptr(w_down), _ptr(b_up), _ptr(b_gate),
            _ptr(b_down)))

    def set_expert_f16(self, e, w_up, w_gate, w_down, b_up=None, b_gate=None, b_down=None):
        """w_*: float16 arrays [F,H], [F,H], [H,F]."""
        if w_up is not None:
            w_up, w_gate, w_down = (np.ascontiguousarray(w, dtype=np.float16)
                                    for w in (w_up, w_gate, w_down))
            assert w_up.shape == (self.F, self.H) and w_gate.shape == (self.F, self.H)
            assert w_down.shape == (self.H, self.F)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        self.lib.check(self.lib.dll.csk_layer_set_expert_f16(
            self.h, e, _ptr(w_up), _ptr(w_gate), _ptr(w_down), _ptr(b_up), _ptr(b_gate),
            _ptr(b_down)))

    def set_expert_matrix(self, e, which, ggml_type, data):
        data = _u8(data)
        self.lib.check(self.lib.dll.csk_layer_set_expert_matrix(self.h, e, which, ggml_type, _ptr(data)))

    def export_f16(self, e, which):
        rows, K = (self.H, self.F) if which == W_DOWN else (self.F, self.H)
        out = np.empty((rows, K), np.float16)
        self.lib.check(self.lib.dll.csk_layer_export_f16(self.h, e, which, _ptr(out)))
        return out

    def set_norm(self, w, eps):
        w = _f32(w)
        self.lib.check(self.lib.dll.csk_layer_set_norm(self.h, _ptr(w), eps))

    def fill_synthetic(self, seed, layer_index, scale_lo=117, scale_span=5):
        self.lib.check(self.lib.dll.csk_layer_fill_synthetic(self.h, seed, layer_index, scale_lo,
                                                             scale_span))

    def dequant(self, e, which):
        rows, K = (self.H, self.F) if which == W_DOWN else (self.F, self.H)
        out = np.empty((rows, K), np.float32)
        self.lib.check(self.lib.dll.csk_layer_dequant(self.h, e, which, _ptr(out)))
        return out

    def export(self, e, which):
        rows, K = (self.H, self.F) if which == W_DOWN else (self.F, self.H)
        out = np.empty(rows * (K // 32) * 17, np.uint8)
        self.lib.check(self.lib.dll.csk_layer_export(self.h, e, which, _ptr(out)))
        return out

    def forward_device(self, d_hidden, T, d_out, flags=0):
        self.lib.check(self.lib.dll.csk_moe_forward(self.h, d_hidden, T, d_out, flags))

    def forward_device_noalloc(self, d_hidden, T, d_out, flags=0):
        self.lib.check(self.lib.dll.csk_moe_forward_noalloc(self.h, d_hidden, T, d_out, flags))

    def forward(self, hidden, flags=0, want_pairs=False):
        hidden = _f32(hidden)
        T = hidden.shape[0]
        out = np.empty((T, self.H), np.float32)
        pairs = np.empty((T, self.k, 2), np.float32) if want_pairs else None
        self.lib.check(self.lib.dll.csk_moe_forward_host(self.h, _ptr(hidden), T, _ptr(out),
                                                         _ptr(pairs), flags))
        return (out, pairs) if want_pairs else out

    def last_dispatch(self, T):
        counts = np.empty(self.E, np.int32)
        toks = np.empty(T * self.k, np.int32)
        self.lib.check(self.lib.dll.csk_layer_last_dispatch(self.h, _ptr(counts), _ptr(toks)))
        return counts, toks


def stack_forward(lib, layers, d_hidden, T):
    arr = (_P * len(layers))(*[l.h for l in layers])
    lib.check(lib.dll.csk_moe_stack_forward(arr, len(layers), d_hidden, T))


_lib = None


def load(device=0):
    """Load and initialise the library once per process."""
    global _lib
    if _lib is None:
        _lib = Library().init(device)
    return _lib
