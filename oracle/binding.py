"""ctypes binding of oracle/liboracle.so (and oracle/_ref/libref_mxfp4.so).

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ACT_MODIFIED_SWIGLU, ACT_STANDARD_SWIGLU = 0, 1
OK, ERR_ARG, ERR_RANGE, ERR_ALL_EMPTY = 0, 1, 2, 3
_P = C.c_void_p
_I64 = C.c_int64


def build():
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.uint8)


def _f16(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float16)


class _LayerStruct(C.Structure):
    _fields_ = [("E", _I64), ("k", _I64), ("H", _I64), ("F", _I64),
                ("gate_w", _P), ("gate_b", _P), ("w_up", _P), ("w_gate", _P), ("w_down", _P),
                ("b_up", _P), ("b_gate", _P), ("b_down", _P), ("norm_w", _P),
                ("norm_eps", C.c_float), ("residual", C.c_int), ("sigmoid", C.c_int),
                ("act", C.c_int), ("weight_before_ffn", C.c_int),
                ("w_up16", _P), ("w_gate16", _P), ("w_down16", _P)]


class Oracle:
    def __init__(self):
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        d = self.dll = C.CDLL(path)
        d.orc_e8m0_to_fp32_half.restype = C.c_float
        d.orc_e8m0_to_fp32_half.argtypes = [C.c_uint8]
        d.orc_dequant_mxfp4.restype = None
        d.orc_dequant_mxfp4.argtypes = [_P, _P, _I64]
        for name in ("orc_dequant_q4_k", "orc_dequant_q6_k"):
            getattr(d, name).restype = None
            getattr(d, name).argtypes = [_P, _P, _I64]
        for name in ("orc_q4k_to_fp16", "orc_q6k_to_fp16"):
            getattr(d, name).restype = C.c_int
            getattr(d, name).argtypes = [_P, _P, _I64]
        d.orc_fp32_to_fp16.restype = C.c_uint16
        d.orc_fp32_to_fp16.argtypes = [C.c_float]
        d.orc_router.restype = C.c_int
        d.orc_router.argtypes = [_P, _I64, _I64, _P, _I64, _P, _I64, C.c_int, _P]
        d.orc_router_logits.restype = None
        d.orc_router_logits.argtypes = [_P, _I64, _I64, _P, _I64, _P, _P]
        d.orc_expert_token_mxfp4.restype = C.c_int
        d.orc_expert_token_mxfp4.argtypes = [_P] * 8 + [_I64, _I64, C.c_int]
        d.orc_expert_mlp_mxfp4.restype = C.c_int
        d.orc_expert_mlp_mxfp4.argtypes = [C.c_int, _P, _I64, _I64, _I64] + [_P] * 7 + \
            [_I64, C.c_int, C.c_int, _P, C.POINTER(C.c_int)]
        d.orc_expert_token_f16.restype = C.c_int
        d.orc_expert_token_f16.argtypes = [_P] * 8 + [_I64, _I64, C.c_int]
        d.orc_expert_mlp_f16.restype = C.c_int
        d.orc_expert_mlp_f16.argtypes = [C.c_int, _P, _I64, _I64, _I64] + [_P] * 7 + \
            [_I64, C.c_int, C.c_int, _P, C.POINTER(C.c_int)]
        d.orc_dense_ffn_f16.restype = C.c_int
        d.orc_dense_ffn_f16.argtypes = [_P, _I64, _I64, _I64] + [_P] * 7
        d.orc_matmul_transpose_f16.restype = None
        d.orc_matmul_transpose_f16.argtypes = [_P, _P, _P, _I64, _I64, _I64]
        d.orc_matmul_transpose_f32.restype = None
        d.orc_matmul_transpose_f32.argtypes = [_P, _P, _P, _I64, _I64, _I64]
        d.orc_matmul_transpose_batched.restype = None
        d.orc_matmul_transpose_batched.argtypes = [_P, _I64, _P, _I64, C.c_int, _I64, _P, _I64, _I64, _I64]
        d.orc_dense_ffn_f32.restype = C.c_int
        d.orc_dense_ffn_f32.argtypes = [_P, _I64, _I64, _I64] + [_P] * 7
        d.orc_add_broadcast.restype = C.c_int
        d.orc_add_broadcast.argtypes = [_P, _P, C.c_int, _P, _P, C.c_int, C.c_int, _P, _P]
        d.orc_router_f64.restype = C.c_int
        d.orc_router_f64.argtypes = [_P, _I64, _I64, _P, _I64, _P, _I64, C.c_int, _P, _P]
        d.orc_expert_merge.restype = C.c_int
        d.orc_expert_merge.argtypes = [_P, _I64, _I64, _I64, _I64, C.POINTER(_P), C.c_int, _P]
        d.orc_rmsnorm.restype = None
        d.orc_rmsnorm.argtypes = [_P, _P, _P, _I64, _I64, C.c_float]
        d.orc_rmsnorm_f64.restype = None
        d.orc_rmsnorm_f64.argtypes = [_P, _P, _P, _I64, _I64, C.c_float]
        d.orc_add.restype = None
        d.orc_add.argtypes = [_P, _P, _P, _I64]
        d.orc_moe_layer.restype = C.c_int
        d.orc_moe_layer.argtypes = [C.POINTER(_LayerStruct), _P, _I64, _P, _P, _I64]

    def e8m0(self, x):
        return self.dll.orc_e8m0_to_fp32_half(int(x))

    def dequant(self, blocks, k):
        blocks = _u8(blocks)
        out = np.empty(k, np.float32)
        self.dll.orc_dequant_mxfp4(_p(blocks), _p(out), k)
        return out

    def dequant_kquant(self, kind, blocks, k):
        """kind: "q4_k" (144-byte super-blocks) or "q6_k" (210-byte); k values, fp32."""
        blocks = _u8(blocks)
        out = np.empty(k, np.float32)
        getattr(self.dll, "orc_dequant_" + kind)(_p(blocks), _p(out), k)
        return out

    def kquant_to_fp16(self, kind, blocks, k):
        """The weight provider's widening of a K-quant slice: uint16 bit patterns."""
        blocks = _u8(blocks)
        out = np.empty(k, np.uint16)
        rc = getattr(self.dll, {"q4_k": "orc_q4k_to_fp16", "q6_k": "orc_q6k_to_fp16"}[kind])(_p(blocks), _p(out), k)
        if rc:
            raise ValueError(f"kquant_to_fp16 rc={rc}")
        return out

    def fp32_to_fp16(self, x):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        return np.array([self.dll.orc_fp32_to_fp16(float(v)) for v in x], np.uint16)

    def router(self, hidden, gate_w, gate_b, k, sigmoid=False):
        hidden, gate_w, gate_b = _f32(hidden), _f32(gate_w), _f32(gate_b)
        T, H = hidden.shape
        E = gate_w.shape[0]
        out = np.empty((T, k, 2), np.float32)
        rc = self.dll.orc_router(_p(hidden), T, H, _p(gate_w), E, _p(gate_b), k, int(sigmoid), _p(out))
        if rc:
            raise ValueError(f"orc_router rc={rc}")
        return out

    def router_logits(self, hidden, gate_w, gate_b):
        hidden, gate_w, gate_b = _f32(hidden), _f32(gate_w), _f32(gate_b)
        T, H = hidden.shape
        E = gate_w.shape[0]
        out = np.empty((T, E), np.float32)
        self.dll.orc_router_logits(_p(hidden), T, H, _p(gate_w), E, _p(gate_b), _p(out))
        return out

    def expert_token(self, x, w_up, w_gate, w_down, b_up, b_gate, b_down, H, F, act=0):
        x = _f32(x)
        w_up, w_gate, w_down = _u8(w_up), _u8(w_gate), _u8(w_down)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        out = np.empty(H, np.float32)
        rc = self.dll.orc_expert_token_mxfp4(_p(x), _p(w_up), _p(w_gate), _p(w_down), _p(b_up),
                                             _p(b_gate), _p(b_down), _p(out), H, F, act)
        if rc:
            raise ValueError(f"orc_expert_token_mxfp4 rc={rc}")
        return out

    def expert_mlp(self, expert_id, hidden, F, w_up, w_gate, w_down, b_up, b_gate, b_down, pairs,
                   act=0, weight_before_ffn=False):
        hidden, pairs = _f32(hidden), _f32(pairs)
        w_up, w_gate, w_down = _u8(w_up), _u8(w_gate), _u8(w_down)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        T, H = hidden.shape
        k = pairs.shape[1]
        out = np.empty((T, H), np.float32)
        empty = C.c_int()
        rc = self.dll.orc_expert_mlp_mxfp4(expert_id, _p(hidden), T, H, F, _p(w_up), _p(w_gate),
                                           _p(w_down), _p(b_up), _p(b_gate), _p(b_down), _p(pairs),
                                           k, act, int(weight_before_ffn), _p(out), C.byref(empty))
        if rc:
            raise ValueError(f"orc_expert_mlp_mxfp4 rc={rc}")
        return None if empty.value else out

    def expert_token_f16(self, x, w_up, w_gate, w_down, b_up, b_gate, b_down, act=0):
        """w_* are float16 arrays, row-major [F,H], [F,H], [H,F]."""
        x = _f32(x)
        w_up, w_gate, w_down = _f16(w_up), _f16(w_gate), _f16(w_down)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        F, H = w_up.shape
        out = np.empty(H, np.float32)
        rc = self.dll.orc_expert_token_f16(_p(x), _p(w_up), _p(w_gate), _p(w_down), _p(b_up),
                                           _p(b_gate), _p(b_down), _p(out), H, F, act)
        if rc:
            raise ValueError(f"orc_expert_token_f16 rc={rc}")
        return out

    def expert_mlp_f16(self, expert_id, hidden, w_up, w_gate, w_down, b_up, b_gate, b_down, pairs,
                       act=0, weight_before_ffn=False):
        hidden, pairs = _f32(hidden), _f32(pairs)
        w_up, w_gate, w_down = _f16(w_up), _f16(w_gate), _f16(w_down)
        b_up, b_gate, b_down = _f32(b_up), _f32(b_gate), _f32(b_down)
        T, H = hidden.shape
        F = w_up.shape[0]
        k = pairs.shape[1]
        out = np.empty((T, H), np.float32)
        empty = C.c_int()
        rc = self.dll.orc_expert_mlp_f16(expert_id, _p(hidden), T, H, F, _p(w_up), _p(w_gate),
                                         _p(w_down), _p(b_up), _p(b_gate), _p(b_down), _p(pairs),
                                         k, act, int(weight_before_ffn), _p(out), C.byref(empty))
        if rc:
            raise ValueError(f"orc_expert_mlp_f16 rc={rc}")
        return None if empty.value else out

    def dense_ffn_f16(self, hidden, w_gate, w_up, w_down, b_gate=None, b_up=None, b_down=None):
        """dense_ffn_node: hidden [T,H]; float16 w_gate/w_up [F,H], w_down [H,F]."""
        hidden = _f32(hidden)
        w_gate, w_up, w_down = _f16(w_gate), _f16(w_up), _f16(w_down)
        b_gate, b_up, b_down = _f32(b_gate), _f32(b_up), _f32(b_down)
        T, H = hidden.shape
        F = w_gate.shape[0]
        out = np.empty((T, H), np.float32)
        rc = self.dll.orc_dense_ffn_f16(_p(hidden), T, H, F, _p(w_gate), _p(w_up), _p(w_down), _p(b_gate),
                                        _p(b_up), _p(b_down), _p(out))
        if rc:
            raise ValueError(f"orc_dense_ffn_f16 rc={rc}")
        return out

    def matmul_transpose_f16(self, a, b):
        """matmul_transpose_mixed_node with a float16 weight: a [M,K] f32, b [N,K] f16 -> [M,N]."""
        a, b = _f32(a), _f16(b)
        M, K = a.shape
        N = b.shape[0]
        out = np.empty((M, N), np.float32)
        self.dll.orc_matmul_transpose_f16(_p(a), _p(b), _p(out), M, K, N)
        return out

    def matmul_transpose_f32(self, a, b):
        """matmul_transpose_mixed_node with a float32 weight: a [M,K], b [N,K] -> [M,N]."""
        a, b = _f32(a), _f32(b)
        M, K = a.shape
        N = b.shape[0]
        out = np.empty((M, N), np.float32)
        self.dll.orc_matmul_transpose_f32(_p(a), _p(b), _p(out), M, K, N)
        return out

    def matmul_transpose_batched(self, a, b):
        """a [*, M, K] float32, b [*, N, K] float16 or float32; the node's batch rule
        (output matrix i pairs matrix i % n_a of a with matrix i % n_b of b)."""
        a = _f32(a)
        b = _f16(b) if b.dtype == np.float16 else _f32(b)
        M, K = a.shape[-2:]
        N = b.shape[-2]
        batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
        n_out = int(np.prod(batch, dtype=np.int64))
        n_a, n_b = a.size // (M * K), b.size // (N * K)
        out = np.empty(tuple(batch) + (M, N), np.float32)
        self.dll.orc_matmul_transpose_batched(_p(a), n_a, _p(b), n_b, int(b.dtype == np.float16), n_out,
                                              _p(out), M, K, N)
        return out

    def dense_ffn_f32(self, hidden, w_gate, w_up, w_down, b_gate=None, b_up=None, b_down=None):
        """dense_ffn_node with FLOAT32 weights: hidden [T,H]; w_gate/w_up [F,H], w_down [H,F]."""
        hidden = _f32(hidden)
        w_gate, w_up, w_down = _f32(w_gate), _f32(w_up), _f32(w_down)
        b_gate, b_up, b_down = _f32(b_gate), _f32(b_up), _f32(b_down)
        T, H = hidden.shape
        F = w_gate.shape[0]
        out = np.empty((T, H), np.float32)
        rc = self.dll.orc_dense_ffn_f32(_p(hidden), T, H, F, _p(w_gate), _p(w_up), _p(w_down), _p(b_gate),
                                        _p(b_up), _p(b_down), _p(out))
        if rc:
            raise ValueError(f"orc_dense_ffn_f32 rc={rc}")
        return out

    _ADD_DTYPES = {np.dtype(np.float32): 0, np.dtype(np.float64): 1, np.dtype(np.int32): 2, np.dtype(np.int64): 3}

    def add_broadcast(self, a, b):
        """add_node over two arrays of one element type; None when the shapes do not broadcast."""
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        assert a.dtype == b.dtype
        nd = max(a.ndim, b.ndim)
        sa = np.array(a.shape, np.int64)
        sb = np.array(b.shape, np.int64)
        oshape = np.zeros(max(nd, 1), np.int64)
        # size the output before the call: the shape is a function of the inputs' shapes alone
        try:
            shape = np.broadcast_shapes(a.shape, b.shape)
        except ValueError:
            shape = (0,)
        out = np.empty(shape, a.dtype)
        rc = self.dll.orc_add_broadcast(_p(a), _p(sa), a.ndim, _p(b), _p(sb), b.ndim,
                                        self._ADD_DTYPES[a.dtype], _p(out), _p(oshape))
        if rc:
            return None
        assert tuple(oshape[:nd]) == tuple(shape), (oshape, shape)
        return out

    def router_f64(self, hidden, gate_w, gate_b, k, sigmoid=False, want_logits=False):
        hidden = np.ascontiguousarray(hidden, np.float64)
        gate_w = np.ascontiguousarray(gate_w, np.float64)
        gate_b = _f32(gate_b)
        T, H = hidden.shape
        E = gate_w.shape[0]
        out = np.empty((T, k, 2), np.float32)
        logits = np.empty((T, E), np.float64) if want_logits else None
        rc = self.dll.orc_router_f64(_p(hidden), T, H, _p(gate_w), E, _p(gate_b), k, int(sigmoid),
                                     _p(out), _p(logits))
        if rc:
            raise ValueError(f"orc_router_f64 rc={rc}")
        return (out, logits) if want_logits else out

    def expert_merge(self, pairs, expert_outs, H, pre_weighted=False):
        pairs = _f32(pairs)
        T, k = pairs.shape[:2]
        E = len(expert_outs)
        keep = [_f32(a) for a in expert_outs]
        arr = (_P * E)(*[_p(a) for a in keep])
        out = np.empty((T, H), np.float32)
        rc = self.dll.orc_expert_merge(_p(pairs), T, k, E, H, arr, int(pre_weighted), _p(out))
        return rc, out

    def rmsnorm(self, x, w, eps):
        x, w = _f32(x), _f32(w)
        T, H = x.shape
        out = np.empty((T, H), np.float32)
        self.dll.orc_rmsnorm(_p(x), _p(w), _p(out), T, H, eps)
        return out

    def rmsnorm_f64(self, x, w, eps):
        x = np.ascontiguousarray(x, np.float64)
        w = np.ascontiguousarray(w, np.float64)
        T, H = x.shape
        out = np.empty((T, H), np.float64)
        self.dll.orc_rmsnorm_f64(_p(x), _p(w), _p(out), T, H, eps)
        return out

    def add(self, a, b):
        a, b = _f32(a), _f32(b)
        out = np.empty(a.shape, np.float32)
        self.dll.orc_add(_p(a), _p(b), _p(out), a.size)
        return out

    def moe_layer(self, hidden, E, k, H, F, gate_w, gate_b, w_up, w_gate, w_down, b_up, b_gate,
                  b_down, norm_w=None, norm_eps=1e-5, residual=False, sigmoid=False, act=0,
                  weight_before_ffn=False, max_tokens=-1):
        """w_up/w_gate/w_down: uint8 arrays holding all E experts back to back (MXFP4 blocks),
        or float16 arrays [E,F,H], [E,F,H], [E,H,F] (fp16 experts)."""
        hidden = _f32(hidden)
        f16 = getattr(w_up, "dtype", None) == np.float16
        wconv = _f16 if f16 else _u8
        keep = [_f32(gate_w), _f32(gate_b), wconv(w_up), wconv(w_gate), wconv(w_down), _f32(b_up),
                _f32(b_gate), _f32(b_down), _f32(norm_w)]
        ptrs = [_p(a) for a in keep]
        w16 = ptrs[2:5] if f16 else [None, None, None]
        if f16:
            ptrs[2:5] = [None, None, None]
        L = _LayerStruct(E, k, H, F, *ptrs, norm_eps, int(residual), int(sigmoid),
                         act, int(weight_before_ffn), *w16)
        T = hidden.shape[0]
        out = np.zeros((T, H), np.float32)
        pairs = np.empty((T, k, 2), np.float32)
        rc = self.dll.orc_moe_layer(C.byref(L), _p(hidden), T, _p(out), _p(pairs), max_tokens)
        if rc:
            raise ValueError(f"orc_moe_layer rc={rc}")
        return out, pairs


class RefCodec:
    """The reference's own MXFP4 codec, when oracle/_ref was built."""

    def __init__(self):
        path = os.path.join(_HERE, "_ref", "libref_mxfp4.so")
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        d = self.dll = C.CDLL(path)
        d.ref_e8m0_to_fp32_half.restype = C.c_float
        d.ref_e8m0_to_fp32_half.argtypes = [C.c_uint8]
        d.ref_dequantize_block_mxfp4.restype = None
        d.ref_dequantize_block_mxfp4.argtypes = [_P, _P, _I64]
        self.has_kquant = hasattr(d, "ref_q4k_to_fp16")
        if self.has_kquant:
            for name in ("ref_dequantize_block_q4_K", "ref_dequantize_block_q6_K", "ref_q4k_to_fp16",
                         "ref_q6k_to_fp16"):
                getattr(d, name).restype = None
                getattr(d, name).argtypes = [_P, _P, _I64]
            d.ref_fp32_to_fp16.restype = C.c_uint16
            d.ref_fp32_to_fp16.argtypes = [C.c_float]

    def e8m0(self, x):
        return self.dll.ref_e8m0_to_fp32_half(int(x))

    def dequant(self, blocks, k):
        blocks = _u8(blocks)
        out = np.empty(k, np.float32)
        self.dll.ref_dequantize_block_mxfp4(_p(blocks), _p(out), k)
        return out

    def dequant_kquant(self, kind, blocks, k):
        blocks = _u8(blocks)
        out = np.empty(k, np.float32)
        getattr(self.dll, {"q4_k": "ref_dequantize_block_q4_K", "q6_k": "ref_dequantize_block_q6_K"}[kind])(
            _p(blocks), _p(out), k)
        return out

    def kquant_to_fp16(self, kind, blocks, k):
        blocks = _u8(blocks)
        out = np.empty(k, np.uint16)
        getattr(self.dll, {"q4_k": "ref_q4k_to_fp16", "q6_k": "ref_q6k_to_fp16"}[kind])(_p(blocks), _p(out), k)
        return out

    def fp32_to_fp16(self, x):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        return np.array([self.dll.ref_fp32_to_fp16(float(v)) for v in x], np.uint16)


class RefGguf:
    """The reference's own GGUF readers (gguf_loader / gguf_multi_loader), when oracle/_ref
    was built.  `paths`: one file or the shards of a split checkpoint."""

    def __init__(self, paths):
        path = os.path.join(_HERE, "_ref", "libref_gguf.so")
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.dll = C.CDLL(path)
        self.dll.ref_gguf_open.restype = C.c_void_p
        self.dll.ref_gguf_open.argtypes = [C.POINTER(C.c_char_p), C.c_int64]
        self.dll.ref_gguf_close.argtypes = [C.c_void_p]
        self.dll.ref_gguf_tensor_count.restype = C.c_int64
        self.dll.ref_gguf_tensor_count.argtypes = [C.c_void_p]
        self.dll.ref_gguf_version.restype = C.c_uint32
        self.dll.ref_gguf_version.argtypes = [C.c_void_p]
        self.dll.ref_gguf_tensor_name.argtypes = [C.c_void_p, C.c_int64, C.c_char_p, C.c_size_t]
        self.dll.ref_gguf_tensor_info.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(C.c_int32),
                                                  C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                                  C.POINTER(C.c_uint64), C.POINTER(C.c_int32)]
        self.dll.ref_gguf_get_u32.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_uint32)]
        self.dll.ref_gguf_get_str.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_size_t]
        if isinstance(paths, (str, bytes, os.PathLike)):
            paths = [paths]
        arr = (C.c_char_p * len(paths))(*[os.fsencode(p) for p in paths])
        self.h = self.dll.ref_gguf_open(arr, len(paths))

    @property
    def loaded(self):
        return bool(self.h)

    def close(self):
        if self.h:
            self.dll.ref_gguf_close(self.h)
            self.h = None

    def version(self):
        return self.dll.ref_gguf_version(self.h)

    def tensor_names(self):
        buf = C.create_string_buffer(512)
        out = []
        for i in range(self.dll.ref_gguf_tensor_count(self.h)):
            assert self.dll.ref_gguf_tensor_name(self.h, i, buf, 512) == 0
            out.append(buf.value.decode())
        return out

    def tensor_info(self, name):
        t, nd, off, nb, sh = C.c_uint32(), C.c_int32(), C.c_uint64(), C.c_uint64(), C.c_int32()
        dims = (C.c_uint64 * 4)()
        if self.dll.ref_gguf_tensor_info(self.h, name.encode(), C.byref(t), C.byref(nd), dims, C.byref(off),
                                         C.byref(nb), C.byref(sh)) != 0:
            return None
        return dict(type=t.value, dims=list(dims)[:nd.value], offset=off.value, nbytes=nb.value, shard=sh.value)

    def get_u32(self, key):
        v = C.c_uint32()
        return v.value if self.dll.ref_gguf_get_u32(self.h, key.encode(), C.byref(v)) == 0 else None

    def get_str(self, key):
        buf = C.create_string_buffer(1024)
        return buf.value.decode() if self.dll.ref_gguf_get_str(self.h, key.encode(), buf, 1024) == 0 else None
