"""ctypes binding of libisp_oracle.so (the C oracle) on numpy arrays.

TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels, never the thing measured or shipped.

All functions work on C-contiguous numpy arrays.  In-place oracle functions copy their inputs and
return the results, so callers keep their originals.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ISP_ORACLE_LIB names another build of the same source (the sanitizer build of `make -C oracle asan`)
_SO = os.environ.get("ISP_ORACLE_LIB") or os.path.join(_HERE, "libisp_oracle.so")

NORM_RESIDUAL_EXCLUDES_BIAS = 1


def build(force=False):
    """Compile the oracle with gcc (seconds).  Returns the path of the shared library."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _SO


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _elem_dtype(a):
    if a.dtype == np.float16:
        return "f16"
    if a.dtype == np.float32:
        return "f32"
    raise TypeError("oracle handles float16 and float32 only, got %s" % a.dtype)


class Oracle:
    def __init__(self, path=_SO):
        if not os.path.exists(path):
            build()
        self.lib = C.CDLL(path)
        L = self.lib
        vp, i, f, u, sz = C.c_void_p, C.c_int, C.c_float, C.c_uint, C.c_size_t
        L.isp_oracle_set_threads.argtypes = [i]
        L.isp_oracle_set_threads.restype = i
        L.isp_oracle_max_threads.restype = i
        L.isp_oracle_h2f.argtypes = [C.c_uint16]
        L.isp_oracle_h2f.restype = f
        L.isp_oracle_f2h.argtypes = [f]
        L.isp_oracle_f2h.restype = C.c_uint16
        L.isp_oracle_h2f_array.argtypes = [vp, vp, sz]
        L.isp_oracle_f2h_array.argtypes = [vp, vp, sz]
        L.isp_oracle_embedding.argtypes = [vp, vp, vp, i, i, i]
        L.isp_oracle_cal_padding_offset.argtypes = [vp, vp, vp, i, i]
        for n in ("f32", "f16"):
            getattr(L, "isp_oracle_fused_norm_" + n).argtypes = [vp, vp, vp, vp, f, i, i, u]
            getattr(L, "isp_oracle_qkv_rope_" + n).argtypes = [vp] * 8 + [i] * 7 + [f]
            getattr(L, "isp_oracle_swiglu_" + n).argtypes = [vp, vp, i, i]
            getattr(L, "isp_oracle_rope_decode_" + n).argtypes = [vp, i, i, i, i, i, i, f]
        L.isp_oracle_transpose_remove_padding.argtypes = [vp, vp, vp, i, i, i, i, i, i]
        L.isp_oracle_concat_kv.argtypes = [vp, vp, sz, vp, vp, i, i, i, i, i, i]
        L.isp_oracle_repeat_kv.argtypes = [vp, vp, sz, vp, i, i, i, i, i, i, i]

    # ---- housekeeping
    def set_threads(self, n):
        return self.lib.isp_oracle_set_threads(int(n))

    def max_threads(self):
        return self.lib.isp_oracle_max_threads()

    # ---- fp16 conversion
    def h2f(self, h):
        h = np.ascontiguousarray(h, dtype=np.uint16)
        out = np.empty(h.shape, np.float32)
        self.lib.isp_oracle_h2f_array(_ptr(h), _ptr(out), h.size)
        return out

    def f2h(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape, np.uint16)
        self.lib.isp_oracle_f2h_array(_ptr(x), _ptr(out), x.size)
        return out

    # ---- hot path
    def embedding(self, ids, table):
        ids = _c(ids, np.int32)
        table = np.ascontiguousarray(table)
        tokens, hidden = ids.shape[0], table.shape[1]
        out = np.empty((tokens, hidden), table.dtype)
        self.lib.isp_oracle_embedding(_ptr(ids), _ptr(out), _ptr(table), tokens, hidden,
                                      table.dtype.itemsize)
        return out

    def cal_padding_offset(self, input_lengths, max_q_len, fill=0):
        lens = _c(input_lengths, np.int32)
        batch = lens.shape[0]
        padding_offset = np.full((batch, max_q_len), fill, np.int32)
        cum = np.full((batch + 1,), fill, np.int32)
        self.lib.isp_oracle_cal_padding_offset(_ptr(padding_offset), _ptr(cum), _ptr(lens), batch,
                                               max_q_len)
        return padding_offset, cum

    def fused_norm(self, residual, decoder_out, bias, gamma, eps, flags=0):
        """Returns (residual_new or None, normalised_out)."""
        kind = _elem_dtype(decoder_out)
        out = np.array(decoder_out, copy=True, order="C")
        rsd = None if residual is None else np.array(residual, copy=True, order="C")
        bias = None if bias is None else np.ascontiguousarray(bias, dtype=out.dtype)
        gamma = np.ascontiguousarray(gamma, dtype=out.dtype)
        tokens, hidden = out.shape
        getattr(self.lib, "isp_oracle_fused_norm_" + kind)(
            _ptr(rsd), _ptr(out), _ptr(bias), _ptr(gamma), float(eps), tokens, hidden, int(flags))
        return rsd, out

    def rmsnorm(self, x, gamma, eps):
        return self.fused_norm(None, x, None, gamma, eps)[1]

    def qkv_rope(self, qkv, bias, padding_offset, history_length, input_length, batch, seq_len,
                 head_num, kv_head_num, rotary_dim, rotary_base, fill=0.0):
        """qkv [token_num, head_num + 2 kv_head_num, head_size] -> (q, k, v) padded, positions that
        the step does not write hold `fill`."""
        kind = _elem_dtype(qkv)
        qkv = np.ascontiguousarray(qkv)
        token_num, qkv_heads, head_size = qkv.shape
        assert qkv_heads == head_num + 2 * kv_head_num
        bias = None if bias is None else np.ascontiguousarray(bias, dtype=qkv.dtype)
        po = _c(padding_offset, np.int32).reshape(-1)
        hist = _c(history_length, np.int32)
        ilen = _c(input_length, np.int32)
        q = np.full((batch, head_num, seq_len, head_size), fill, qkv.dtype)
        k = np.full((batch, kv_head_num, seq_len, head_size), fill, qkv.dtype)
        v = np.full((batch, kv_head_num, seq_len, head_size), fill, qkv.dtype)
        getattr(self.lib, "isp_oracle_qkv_rope_" + kind)(
            _ptr(q), _ptr(k), _ptr(v), _ptr(qkv), _ptr(bias), _ptr(po), _ptr(hist), _ptr(ilen),
            batch, seq_len, token_num, head_num, kv_head_num, head_size, int(rotary_dim),
            float(rotary_base))
        return q, k, v

    def swiglu(self, x):
        kind = _elem_dtype(x)
        x = np.ascontiguousarray(x)
        tokens, two, inter = x.shape
        assert two == 2
        out = np.empty((tokens, inter), x.dtype)
        getattr(self.lib, "isp_oracle_swiglu_" + kind)(_ptr(x), _ptr(out), tokens, inter)
        return out

    # ---- callers either side of the path
    def rope_decode(self, qkv, head_num, kv_head_num, step, rotary_dim, rotary_base):
        kind = _elem_dtype(qkv)
        out = np.array(qkv, copy=True, order="C")
        batch, qkv_heads, head_size = out.shape
        assert qkv_heads == head_num + 2 * kv_head_num
        getattr(self.lib, "isp_oracle_rope_decode_" + kind)(
            _ptr(out), batch, head_num, kv_head_num, head_size, int(step), int(rotary_dim),
            float(rotary_base))
        return out

    def transpose_remove_padding(self, src, padding_offset, token_num):
        src = np.ascontiguousarray(src)
        batch, head_num, seq_len, head_size = src.shape
        po = _c(padding_offset, np.int32).reshape(-1)
        dst = np.empty((token_num, head_num, head_size), src.dtype)
        self.lib.isp_oracle_transpose_remove_padding(_ptr(src), _ptr(dst), _ptr(po), batch,
                                                     head_num, seq_len, head_size, token_num,
                                                     src.dtype.itemsize)
        return dst

    def concat_kv(self, src, cache, layer, cur_query_length, history_length):
        """cache [layers, batch, kv_head_num, max_seq_len, head_size]; returns the updated copy."""
        src = np.ascontiguousarray(src)
        cache = np.array(cache, copy=True, order="C")
        batch, kv_head_num, max_q_len, head_size = src.shape
        max_seq_len = cache.shape[3]
        layer_offset = layer * batch * kv_head_num * max_seq_len * head_size
        cur = _c(cur_query_length, np.int32)
        hist = _c(history_length, np.int32)
        self.lib.isp_oracle_concat_kv(_ptr(src), _ptr(cache), layer_offset, _ptr(cur), _ptr(hist),
                                      batch, kv_head_num, max_q_len, max_seq_len, head_size,
                                      src.dtype.itemsize)
        return cache

    def repeat_kv(self, cache, layer, context_length, head_num, max_k_len, fill=0.0):
        cache = np.ascontiguousarray(cache)
        _, batch, kv_head_num, max_seq_len, head_size = cache.shape
        ctx = _c(context_length, np.int32)
        dst = np.full((batch, head_num, max_k_len, head_size), fill, cache.dtype)
        layer_offset = layer * batch * kv_head_num * max_seq_len * head_size
        self.lib.isp_oracle_repeat_kv(_ptr(cache), _ptr(dst), layer_offset, _ptr(ctx), batch,
                                      head_num, kv_head_num, max_seq_len, max_k_len, head_size,
                                      cache.dtype.itemsize)
        return dst


_ORACLE = None


def load():
    global _ORACLE
    if _ORACLE is None:
        _ORACLE = Oracle()
    return _ORACLE
