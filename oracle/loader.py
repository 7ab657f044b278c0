"""ctypes bindings of liboracle.so -- TEST INFRASTRUCTURE, not part of the product.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module.
All arrays are C-contiguous numpy arrays (float32 / int64 / int8 / int32).
"""
import ctypes
import glob
import os
import subprocess

import numpy as np

# MKL must use the GNU OpenMP layer: the oracle (and usually torch) already run on libgomp.
os.environ.setdefault("MKL_THREADING_LAYER", "GNU")

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "liboracle.so")

c_float_p = ctypes.POINTER(ctypes.c_float)
c_i64_p = ctypes.POINTER(ctypes.c_int64)
c_i32_p = ctypes.POINTER(ctypes.c_int32)
c_i8_p = ctypes.POINTER(ctypes.c_int8)
i64 = ctypes.c_int64


def build():
    subprocess.run(["make", "-C", _DIR, "-s", "-B"], check=True)
    return _LIB_PATH


class LayerWeights(ctypes.Structure):
    _fields_ = [(n, c_float_p) for n in (
        "qkv_w", "qkv_b", "attn_out_w", "attn_out_b", "attn_ln_g", "attn_ln_b",
        "inter_w", "inter_b", "out_w", "out_b", "out_ln_g", "out_ln_b")]


def _fp(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags.c_contiguous, (a.dtype, a.flags)
    return a.ctypes.data_as(c_float_p)


def _ip(a):
    if a is None:
        return None
    assert a.dtype == np.int64 and a.flags.c_contiguous
    return a.ctypes.data_as(c_i64_p)


class Oracle:
    """Thin numpy-level wrapper; each method mirrors one exported oracle_* function."""

    def __init__(self, blas="auto"):
        if not os.path.exists(_LIB_PATH):
            build()
        self.lib = ctypes.CDLL(_LIB_PATH)
        L = self.lib
        L.oracle_blas_name.restype = ctypes.c_char_p
        L.oracle_load_blas.argtypes = [ctypes.c_char_p, ctypes.c_int]
        L.oracle_quantize_tensor_i8.restype = ctypes.c_float
        L.oracle_max_threads.restype = ctypes.c_int
        self._keep = []
        if blas == "auto":
            self.load_best_blas()

    # ---- BLAS selection: MKL, system OpenBLAS, the OpenBLAS inside the NumPy wheel ----
    def _blas_agrees_with_builtin(self):
        """Multi-threaded sgemm self-check: a BLAS whose threading layer clashes with an OpenMP
        runtime already in the process (MKL's Intel layer next to libgomp) returns garbage."""
        rng = np.random.default_rng(0)
        A = rng.standard_normal((1024, 512), np.float32)
        B = rng.standard_normal((512, 768), np.float32)
        got = self.matmul(A, B)
        return bool(np.abs(got - A @ B).max() < 1e-2)

    def load_best_blas(self):
        cands = [(p, 0) for p in ("/opt/conda/lib/libmkl_rt.so", "/opt/conda/lib/libmkl_rt.so.2",
                                  "libmkl_rt.so", "libopenblas.so", "libopenblas.so.0")]
        cands += [(p, 1) for p in glob.glob(os.path.join(os.path.dirname(np.__file__), "..", "numpy.libs",
                                                         "libscipy_openblas64_*.so"))]
        for path, kind in cands:
            if self.lib.oracle_load_blas(path.encode(), kind) == 0 and self._blas_agrees_with_builtin():
                return self.blas_name()
        self.lib.oracle_use_builtin_blas()
        return self.blas_name()

    def use_builtin_blas(self):
        self.lib.oracle_use_builtin_blas()

    def blas_name(self):
        return self.lib.oracle_blas_name().decode()

    def set_num_threads(self, n):
        self.lib.oracle_set_num_threads(int(n))

    def max_threads(self):
        return self.lib.oracle_max_threads()

    # ---- kernels ----
    def matmul(self, A, B, b_trans=False, alpha=1.0, beta=0.0, C=None):
        M, K = A.shape
        N = B.shape[0] if b_trans else B.shape[1]
        if C is None:
            C = np.zeros((M, N), np.float32)
        self.lib.oracle_matmul(_fp(A), _fp(B), _fp(C), i64(M), i64(N), i64(K), int(b_trans),
                               ctypes.c_float(alpha), ctypes.c_float(beta))
        return C

    def batch_matmul(self, A, B, b_trans=False, alpha=1.0, beta=0.0, C=None):
        batch = int(np.prod(A.shape[:-2]))
        M, K = A.shape[-2:]
        N = B.shape[-2] if b_trans else B.shape[-1]
        if C is None:
            C = np.zeros(A.shape[:-2] + (M, N), np.float32)
        self.lib.oracle_batch_matmul(_fp(A), _fp(B), _fp(C), i64(batch), i64(M), i64(N), i64(K), int(b_trans),
                                     ctypes.c_float(alpha), ctypes.c_float(beta))
        return C

    def split_add_bias_transpose(self, x, bias, B, S, h, d):
        q, k, v = (np.empty((B, h, S, d), np.float32) for _ in range(3))
        self.lib.oracle_split_add_bias_transpose(_fp(x), _fp(bias), _fp(q), _fp(k), _fp(v), i64(B), i64(S), i64(h), i64(d))
        return q, k, v

    def split_add_bias_transpose_pad(self, x, bias, lens, h, d):
        lens = np.ascontiguousarray(lens, np.int64)
        B, maxS = len(lens), int(lens.max())
        q, k, v = (np.empty((B, h, maxS, d), np.float32) for _ in range(3))
        self.lib.oracle_split_add_bias_transpose_pad(_fp(x), _fp(bias), _fp(q), _fp(k), _fp(v), _ip(lens), i64(B),
                                                     i64(maxS), i64(h), i64(d))
        return q, k, v

    def transpose_for_score(self, x):
        B, h, S, d = x.shape
        out = np.empty((B, S, h, d), np.float32)
        self.lib.oracle_transpose_for_score(_fp(x), _fp(out), i64(B), i64(S), i64(h), i64(d))
        return out

    def transpose_for_score_pad(self, x, lens):
        lens = np.ascontiguousarray(lens, np.int64)
        B, h, maxS, d = x.shape
        out = np.empty((int(lens.sum()), h, d), np.float32)
        self.lib.oracle_transpose_for_score_pad(_fp(x), _fp(out), _ip(lens), i64(B), i64(maxS), i64(h), i64(d))
        return out

    def apply_mask_and_softmax(self, qk, mask, scale=1.0, is_2d=True):
        qk = np.array(qk, np.float32, order="C")
        B, h, F, T = qk.shape
        self.lib.oracle_apply_mask_and_softmax(_fp(qk), _fp(mask), i64(B), i64(h), i64(F), i64(T),
                                               ctypes.c_float(scale), int(is_2d))
        return qk

    def layer_norm(self, x, gamma, beta, eps=1e-12):
        x = np.array(x, np.float32, order="C")
        n = x.shape[-1]
        self.lib.oracle_layer_norm(_fp(x), _fp(gamma), _fp(beta), i64(x.size // n), i64(n), ctypes.c_float(eps))
        return x

    def add_bias_layer_norm(self, out, inp, bias, gamma, beta, eps=1e-12):
        out = np.array(out, np.float32, order="C")
        n = out.shape[-1]
        self.lib.oracle_add_bias_layer_norm(_fp(out), _fp(inp), _fp(bias), _fp(gamma), _fp(beta), i64(out.size // n),
                                            i64(n), ctypes.c_float(eps))
        return out

    def add_bias_act(self, out, bias, act=0):
        out = np.array(out, np.float32, order="C")
        n = out.shape[-1]
        self.lib.oracle_add_bias_act(_fp(out), _fp(bias), i64(out.size // n), i64(n), int(act))
        return out

    def lookup_embedding(self, table, ids, out=None, add=False):
        ids = np.ascontiguousarray(ids, np.int64)
        vocab, hidden = table.shape
        if out is None:
            out = np.zeros(ids.shape + (hidden,), np.float32)
        rc = self.lib.oracle_lookup_embedding(_fp(out), _fp(table), _ip(ids), i64(ids.size), i64(hidden), i64(vocab),
                                              int(add))
        if rc != 0:
            raise IndexError("embedding id out of index")
        return out

    def prepare_bert_masks(self, B, S, att_mask=None, seq_type=None, pos_ids=None):
        has = [x is not None for x in (att_mask, seq_type, pos_ids)]
        att_mask = np.ascontiguousarray(att_mask, np.int64) if has[0] else np.empty((B, S), np.int64)
        seq_type = np.ascontiguousarray(seq_type, np.int64) if has[1] else np.empty((B, S), np.int64)
        pos_ids = np.ascontiguousarray(pos_ids, np.int64) if has[2] else np.empty((B, S), np.int64)
        ext = np.empty((B, 1, 1, S), np.float32)
        self.lib.oracle_prepare_bert_masks(i64(B), i64(S), _ip(att_mask), int(has[0]), _ip(seq_type), int(has[1]),
                                           _ip(pos_ids), int(has[2]), _fp(ext))
        return att_mask, seq_type, pos_ids, ext

    def bert_embedding(self, ids, pos_ids, type_ids, word, pos, typ, gamma, beta):
        ids = np.ascontiguousarray(ids, np.int64)
        out = np.empty(ids.shape + (word.shape[1],), np.float32)
        rc = self.lib.oracle_bert_embedding(_fp(out), _ip(ids), _ip(np.ascontiguousarray(pos_ids, np.int64)),
                                            _ip(np.ascontiguousarray(type_ids, np.int64)), _fp(word), _fp(pos),
                                            _fp(typ), _fp(gamma), _fp(beta), i64(ids.size), i64(word.shape[1]),
                                            i64(word.shape[0]), i64(pos.shape[0]), i64(typ.shape[0]))
        if rc != 0:
            raise IndexError("embedding id out of index")
        return out

    # ---- layers ----
    def pack_layer(self, w):
        """w: dict of float32 arrays with the LayerWeights field names."""
        s = LayerWeights()
        for name, _ in LayerWeights._fields_:
            arr = np.ascontiguousarray(w[name], np.float32)
            self._keep.append(arr)
            setattr(s, name, _fp(arr))
        return s

    def bert_attention(self, x, mask, w, heads):
        B, S, H = x.shape
        out = np.empty((B, S, H), np.float32)
        attn = np.empty((B, heads, S, S), np.float32)
        lw = self.pack_layer(w)
        self.lib.oracle_bert_attention(_fp(x), _fp(mask), ctypes.byref(lw), i64(B), i64(S), i64(H), i64(heads), _fp(out), _fp(attn))
        return out, attn

    def smart_attention(self, x, mask, w, lens, heads):
        lens = np.ascontiguousarray(lens, np.int64)
        total, H = x.shape[-2:]
        B, maxS = len(lens), int(lens.max())
        out = np.empty((1, total, H), np.float32)
        attn = np.empty((B, heads, maxS, maxS), np.float32)
        lw = self.pack_layer(w)
        self.lib.oracle_smart_attention(_fp(x), _fp(mask), ctypes.byref(lw), _ip(lens), i64(B), i64(H), i64(heads),
                                        _fp(out), _fp(attn))
        return out, attn

    @staticmethod
    def concat(a, b, dim):
        """kernels::Concat<float> (layers/kernels/utils.cpp:33-93): rows of `a` then rows of `b` along
        `dim`; data movement only, so NumPy's routine is the restatement."""
        return np.ascontiguousarray(np.concatenate([a, b], axis=dim), np.float32)

    def add_bias_transpose_for_score(self, x, bias, B, S, h, d):
        """kernels::AddBiasTransposeForScore (layers/kernels/transpose.cpp:194-232): [B,S,h,d] + bias[h*d]
        -> [B,h,S,d].  It is the one-output case of the split kernel, restated through it with two dummy
        thirds so that the arithmetic (one fp32 add) is the oracle's own."""
        x3 = np.zeros((B * S, 3, h * d), np.float32)
        x3[:, 0, :] = np.asarray(x, np.float32).reshape(B * S, h * d)
        b3 = np.concatenate([np.asarray(bias, np.float32), np.zeros(2 * h * d, np.float32)])
        return self.split_add_bias_transpose(x3.reshape(B * S, 3 * h * d), b3, B, S, h, d)[0]

    def multi_headed_attention(self, key, value, query, mask, w, heads, attn_type="self", layer_cache=None,
                               pre_layernorm=False, post_layernorm=False, post_add_input=False):
        """layers::MultiHeadedAttention::operator() (layers/multi_headed_attention.cpp:260-380) with both
        projections paths (:35-164 context, :168-232 self), composed from the oracle's kernels.

        w: dict with q_w,k_w,v_w [H,H] ([in,out]), q_b,k_b,v_b, qkv_w [H,3H], qkv_b, dense_w, dense_b and,
        when a LayerNorm is used, ln_g, ln_b.  layer_cache: dict of float32 arrays or None entries
        (self_keys/self_values/memory_keys/memory_values); it is updated in place like the reference's.
        mask: additive fp32, (B,1,T) or (B,F,T), or None.  Returns (output [B,F,H], attn [B,h,F,T])."""
        f32 = lambda a: np.ascontiguousarray(a, np.float32)
        query = f32(query)
        B, F, H = query.shape
        d = H // heads
        cache = layer_cache if layer_cache is not None else {}
        has = lambda name: cache.get(name) is not None
        q_in = query
        if pre_layernorm:  # :66-80 / :190-199, eps hard-coded 1e-6
            q_in = self.layer_norm(query, w["ln_g"], w["ln_b"], 1e-6)
        if attn_type == "self":
            qkv = self.matmul(q_in.reshape(B * F, H), f32(w["qkv_w"]))
            q, k, v = self.split_add_bias_transpose(qkv, f32(w["qkv_b"]), B, F, heads, d)
            if has("self_keys"):
                k = self.concat(f32(cache["self_keys"]), k, 2)
            if has("self_values"):
                v = self.concat(f32(cache["self_values"]), v, 2)
            if layer_cache:  # non-empty dict: the grown keys/values go back into the cache (:216-229)
                cache["self_keys"], cache["self_values"] = k.copy(), v.copy()
        elif attn_type == "context":
            q = self.add_bias_transpose_for_score(self.matmul(q_in.reshape(B * F, H), f32(w["q_w"])), w["q_b"], B, F, heads, d)
            if has("memory_keys") and has("memory_values"):
                k, v = f32(cache["memory_keys"]), f32(cache["memory_values"])
            else:
                key, value = f32(key), f32(value)
                Tk = key.shape[1]
                k = self.add_bias_transpose_for_score(self.matmul(key.reshape(B * Tk, H), f32(w["k_w"])), w["k_b"], B, Tk, heads, d)
                v = self.add_bias_transpose_for_score(self.matmul(value.reshape(B * Tk, H), f32(w["v_w"])), w["v_b"], B, Tk, heads, d)
                if layer_cache:
                    cache["memory_keys"], cache["memory_values"] = k.copy(), v.copy()
        else:
            raise ValueError("attn_type should be context or self.")
        T = k.shape[2]
        score = self.batch_matmul(q, k, True, 1.0 / np.sqrt(np.float32(d)))
        is_2d = True
        m = None
        if mask is not None:
            m = f32(mask)
            is_2d = m.size == B * T
        attn = self.apply_mask_and_softmax(score, m, 1.0, is_2d)
        ctx = self.transpose_for_score(self.batch_matmul(attn, v, False)).reshape(B * F, H)
        out = self.matmul(ctx, f32(w["dense_w"])).reshape(B, F, H)
        if post_add_input:       # AddInputBias (:371-373)
            out = out + query + f32(w["dense_b"])
        elif post_layernorm:     # AddBiasLayerNorm with the query as residual, eps 1e-12 (:363-369)
            out = self.add_bias_layer_norm(out, query, f32(w["dense_b"]), f32(w["ln_g"]), f32(w["ln_b"]), 1e-12)
        else:                    # AddBias (:360-361)
            out = out + f32(w["dense_b"])
        return f32(out), attn

    def positionwise_ffn(self, x, w1, b1, w2, b2, ln_g, ln_b):
        """layers::PositionwiseFeedForward (layers/positionwise_ffn.cpp:33-77): LayerNorm (eps 1e-12), MatMul,
        AddBiasAct<Relu>, MatMul, AddInputBias.  Weights [in, out]."""
        x = np.ascontiguousarray(x, np.float32)
        B, S, H = x.shape
        normed = self.layer_norm(x, ln_g, ln_b, 1e-12)
        hidden = self.add_bias_act(self.matmul(normed.reshape(B * S, H), np.ascontiguousarray(w1, np.float32)), b1, 2)
        out = self.matmul(hidden, np.ascontiguousarray(w2, np.float32)).reshape(B, S, H)
        return np.ascontiguousarray(out + x + np.asarray(b2, np.float32), np.float32)

    def distill_ffn(self, x, w1, b1, w2, b2, ln_g, ln_b):
        """layers::DistrillFFN (layers/positionwise_ffn.cpp:79-127): MatMul, AddBiasAct<Gelu>, MatMul,
        AddInputBias, LayerNorm (eps 1e-12) -- the last two are exactly AddBiasLayerNorm."""
        x = np.ascontiguousarray(x, np.float32)
        B, S, H = x.shape
        hidden = self.add_bias_act(self.matmul(x.reshape(B * S, H), np.ascontiguousarray(w1, np.float32)), b1, 0)
        out = self.matmul(hidden, np.ascontiguousarray(w2, np.float32)).reshape(B, S, H)
        return self.add_bias_layer_norm(out, x, b2, ln_g, ln_b, 1e-12)

    def bert_layer(self, x, mask, w, heads):
        B, S, H = x.shape
        F = w["inter_w"].shape[1]
        out = np.empty((B, S, H), np.float32)
        attn = np.empty((B, heads, S, S), np.float32)
        lw = self.pack_layer(w)
        self.lib.oracle_bert_layer(_fp(x), _fp(mask), ctypes.byref(lw), i64(B), i64(S), i64(H), i64(heads), i64(F),
                                   _fp(out), _fp(attn))
        return out, attn

    def smart_layer(self, x, mask, w, lens, heads):
        lens = np.ascontiguousarray(lens, np.int64)
        total, H = x.shape[-2:]
        F = w["inter_w"].shape[1]
        B, maxS = len(lens), int(lens.max())
        out = np.empty((1, total, H), np.float32)
        attn = np.empty((B, heads, maxS, maxS), np.float32)
        lw = self.pack_layer(w)
        self.lib.oracle_smart_layer(_fp(x), _fp(mask), ctypes.byref(lw), _ip(lens), i64(B), i64(H), i64(heads), i64(F),
                                    _fp(out), _fp(attn))
        return out, attn

    def bert_encoder(self, x, mask, layers, heads):
        B, S, H = x.shape
        F = layers[0]["inter_w"].shape[1]
        arr = (LayerWeights * len(layers))(*[self.pack_layer(w) for w in layers])
        out = np.empty((B, S, H), np.float32)
        attn = np.empty((B, heads, S, S), np.float32)
        self.lib.oracle_bert_encoder(_fp(x), _fp(mask), arr, i64(len(layers)), i64(B), i64(S), i64(H), i64(heads),
                                     i64(F), _fp(out), _fp(attn))
        return out

    # ---- int8 ----
    def quantize_tensor_i8(self, x):
        x = np.ascontiguousarray(x, np.float32)
        q = np.empty(x.shape, np.int8)
        s = self.lib.oracle_quantize_tensor_i8(_fp(x), q.ctypes.data_as(c_i8_p), i64(x.size))
        return q, float(s)

    def quantize_weight_i8(self, w):
        w = np.ascontiguousarray(w, np.float32)
        N, K = w.shape
        q = np.empty((N, K), np.int8)
        s = np.empty(N, np.float32)
        self.lib.oracle_quantize_weight_i8(_fp(w), q.ctypes.data_as(c_i8_p), _fp(s), i64(N), i64(K))
        return q, s

    def gemm_i8(self, A, B):
        M, K = A.shape
        N = B.shape[0]
        C = np.empty((M, N), np.int32)
        self.lib.oracle_gemm_i8(A.ctypes.data_as(c_i8_p), B.ctypes.data_as(c_i8_p), C.ctypes.data_as(c_i32_p), i64(M),
                                i64(N), i64(K))
        return C

    def dequant_bias(self, acc, act_scale, w_scale, bias):
        M, N = acc.shape
        out = np.empty((M, N), np.float32)
        self.lib.oracle_dequant_bias(acc.ctypes.data_as(c_i32_p), ctypes.c_float(act_scale), _fp(w_scale), _fp(bias),
                                     _fp(out), i64(M), i64(N))
        return out
