"""ctypes bindings for the CPU oracle (oracle/liboracle.so) and, where it has been built, the
compiled reference sampler (oracle/_ref/libgeist_ref_sampler.so).

Test infrastructure only: the shipped library never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

c_float_p = C.POINTER(C.c_float)
c_int32_p = C.POINTER(C.c_int32)


class OracleRng(C.Structure):
    _fields_ = [("state", C.c_uint64)]


class DrawInfo(C.Structure):
    _fields_ = [("boundary_dist", C.c_double), ("mass", C.c_double), ("n_keep", C.c_size_t),
                ("draws", C.c_int)]


class ChainParams(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int), ("top_p", C.c_float),
                ("min_p", C.c_float)]


class SessionSampler(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("top_k", C.c_int),
                ("rng", OracleRng)]


def _fp(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(c_float_p)


def _ip(a):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(c_int32_p)


def build_oracle():
    subprocess.run(["make", "-C", ORACLE_DIR, "-s"], check=True)


def load_oracle(fast=False):
    name = "liboracle_fast.so" if fast else "liboracle.so"
    path = os.path.join(ORACLE_DIR, name)
    if not os.path.exists(path):
        build_oracle()
    lib = C.CDLL(path)
    lib.oracle_rng_next_u64.restype = C.c_uint64
    lib.oracle_rng_next_unit.restype = C.c_float
    lib.oracle_argmax.restype = C.c_int32
    lib.oracle_argmax.argtypes = [C.c_size_t, c_float_p]
    lib.oracle_softmax_into.restype = C.c_double
    lib.oracle_softmax_into.argtypes = [C.c_size_t, c_float_p, C.c_float, c_float_p]
    lib.oracle_softmax_normalised.restype = C.c_double
    lib.oracle_softmax_normalised.argtypes = [C.c_size_t, c_float_p, C.c_float, c_float_p]
    lib.oracle_temperature_u.restype = C.c_int32
    lib.oracle_temperature_u.argtypes = [C.c_size_t, c_float_p, C.c_float, C.c_float,
                                         C.POINTER(DrawInfo)]
    lib.oracle_top_k_u.restype = C.c_int32
    lib.oracle_top_k_u.argtypes = [C.c_size_t, c_float_p, C.c_int, C.c_float, C.c_float,
                                   C.POINTER(DrawInfo)]
    lib.oracle_top_p_u.restype = C.c_int32
    lib.oracle_top_p_u.argtypes = [C.c_size_t, c_float_p, C.c_float, C.c_float, C.c_float,
                                   C.POINTER(DrawInfo)]
    lib.oracle_temperature.restype = C.c_int32
    lib.oracle_temperature.argtypes = [C.c_size_t, c_float_p, C.c_float, C.POINTER(OracleRng)]
    lib.oracle_top_k.restype = C.c_int32
    lib.oracle_top_k.argtypes = [C.c_size_t, c_float_p, C.c_int, C.c_float, C.POINTER(OracleRng)]
    lib.oracle_top_p.restype = C.c_int32
    lib.oracle_top_p.argtypes = [C.c_size_t, c_float_p, C.c_float, C.c_float, C.POINTER(OracleRng)]
    lib.oracle_session_apply_opts.argtypes = [C.POINTER(SessionSampler), C.c_float, C.c_float,
                                              C.c_int, C.c_uint64]
    lib.oracle_session_draws.argtypes = [C.POINTER(SessionSampler), C.c_size_t]
    lib.oracle_softcap_inplace.argtypes = [C.c_size_t, c_float_p, C.c_float]
    lib.oracle_logprob_at.argtypes = [C.c_size_t, c_float_p, C.c_int32]
    lib.oracle_logprob_at.restype = C.c_double
    lib.oracle_propose_drafts_ngram.restype = C.c_size_t
    lib.oracle_propose_drafts_ngram.argtypes = [c_int32_p, C.c_size_t, C.c_int32, C.c_size_t,
                                                C.c_size_t, c_int32_p, C.POINTER(C.c_size_t)]
    lib.oracle_finalize_row.restype = C.c_int32
    lib.oracle_finalize_row.argtypes = [C.POINTER(SessionSampler), C.c_size_t, c_float_p, C.c_float]
    lib.oracle_finalize_batch.argtypes = [C.POINTER(SessionSampler), C.c_size_t, C.c_size_t,
                                          c_float_p, C.c_float, c_int32_p]
    lib.oracle_apply_penalties.argtypes = [C.c_size_t, c_float_p, c_int32_p, C.c_size_t, C.c_float,
                                           C.c_float, C.c_float]
    lib.oracle_sample_chain_u.restype = C.c_int32
    lib.oracle_sample_chain_u.argtypes = [C.c_size_t, c_float_p, C.POINTER(ChainParams), C.c_float,
                                          C.POINTER(DrawInfo)]
    lib.oracle_spec_verify.restype = C.c_int32
    lib.oracle_spec_verify.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_size_t, c_float_p,
                                       C.c_size_t, c_int32_p, c_float_p, C.c_float, c_int32_p]
    lib.oracle_batch_top_k_u.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_size_t, C.c_int,
                                         C.c_float, c_float_p, c_int32_p, C.c_int]
    lib.oracle_batch_chain_u.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_size_t,
                                         C.POINTER(ChainParams), c_int32_p, C.c_size_t, c_int32_p,
                                         C.c_float, C.c_float, C.c_float, c_float_p, c_int32_p,
                                         C.c_int]
    lib.oracle_max_threads.restype = C.c_int
    c_u16_p = C.POINTER(C.c_uint16)
    lib.oracle_f16_to_f32.restype = C.c_float
    lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
    lib.oracle_f32_to_f16.restype = C.c_uint16
    lib.oracle_f32_to_f16.argtypes = [C.c_float]
    lib.oracle_f16_gemv_m1.argtypes = [C.c_size_t, C.c_size_t, c_float_p, c_u16_p, c_float_p]
    c_i8_p = C.POINTER(C.c_int8)
    lib.oracle_f16_to_q8w.argtypes = [C.c_size_t, C.c_size_t, c_u16_p, c_i8_p, c_float_p]
    lib.oracle_q8w_gemv_m1.argtypes = [C.c_size_t, C.c_size_t, c_float_p, c_i8_p, c_float_p,
                                       c_float_p]
    lib.oracle_rmsnorm_rows.argtypes = [C.c_size_t, C.c_size_t, c_float_p, c_float_p, C.c_float,
                                        c_float_p]
    return lib


class Oracle:
    """Thin numpy-facing wrapper."""

    def __init__(self, fast=False):
        self.lib = load_oracle(fast)

    # -- rng
    def rng(self, seed):
        r = OracleRng()
        self.lib.oracle_rng_seed(C.byref(r), C.c_uint64(seed))
        return r

    def next_u64(self, r):
        return int(self.lib.oracle_rng_next_u64(C.byref(r)))

    def next_unit(self, r):
        return float(self.lib.oracle_rng_next_unit(C.byref(r)))

    # -- modes
    def argmax(self, row):
        return int(self.lib.oracle_argmax(row.size, _fp(row)))

    def softmax_into(self, row, t):
        out = np.empty_like(row)
        s = self.lib.oracle_softmax_into(row.size, _fp(row), t, _fp(out))
        return out, float(s)

    def softmax_normalised(self, row, t):
        out = np.empty_like(row)
        s = self.lib.oracle_softmax_normalised(row.size, _fp(row), t, _fp(out))
        return out, float(s)

    def temperature_u(self, row, t, u):
        info = DrawInfo()
        tok = self.lib.oracle_temperature_u(row.size, _fp(row), t, u, C.byref(info))
        return int(tok), info

    def top_k_u(self, row, k, t, u):
        info = DrawInfo()
        tok = self.lib.oracle_top_k_u(row.size, _fp(row), k, t, u, C.byref(info))
        return int(tok), info

    def top_p_u(self, row, p, t, u):
        info = DrawInfo()
        tok = self.lib.oracle_top_p_u(row.size, _fp(row), p, t, u, C.byref(info))
        return int(tok), info

    def chain_u(self, row, u, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0):
        info = DrawInfo()
        prm = ChainParams(temperature, top_k, top_p, min_p)
        tok = self.lib.oracle_sample_chain_u(row.size, _fp(row), C.byref(prm), u, C.byref(info))
        return int(tok), info

    def penalties(self, row, hist, rep, freq, pres):
        out = row.copy()
        hist = np.ascontiguousarray(hist, dtype=np.int32)
        self.lib.oracle_apply_penalties(out.size, _fp(out), _ip(hist), hist.size, rep, freq, pres)
        return out

    def logprob_at(self, row, token):
        row = np.ascontiguousarray(row, dtype=np.float32)
        return float(self.lib.oracle_logprob_at(row.size, _fp(row), int(token)))

    def propose_drafts_ngram(self, history, seed, k_max, max_suffix):
        """-> (drafts as a list, length of the matched suffix)"""
        history = np.ascontiguousarray(history, dtype=np.int32)
        out = np.full(max(int(k_max), 1), -1, dtype=np.int32)
        match = C.c_size_t(99)
        k = self.lib.oracle_propose_drafts_ngram(_ip(history), history.size, int(seed), int(k_max),
                                                 int(max_suffix), _ip(out), C.byref(match))
        return out[:k].tolist(), int(match.value)

    def f16_gemv(self, w_f16, x):
        """w_f16: uint16 [n_out, n_in] (binary16 bit patterns), x: float32 [n_in] or [m, n_in]
        -> float32 [n_out] or [m, n_out], each row of x through oracle_f16_gemv_m1."""
        w = np.ascontiguousarray(w_f16, dtype=np.uint16)
        xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
        n_out, n_in = w.shape
        y = np.empty((xs.shape[0], n_out), dtype=np.float32)
        for m in range(xs.shape[0]):
            self.lib.oracle_f16_gemv_m1(n_out, n_in, _fp(xs[m]),
                                        w.ctypes.data_as(C.POINTER(C.c_uint16)), _fp(y[m]))
        return y[0] if np.ndim(x) == 1 else y

    def f16_to_q8w(self, w_f16):
        w = np.ascontiguousarray(w_f16, dtype=np.uint16)
        n_out, n_in = w.shape
        wq = np.empty((n_out, n_in), dtype=np.int8)
        scales = np.empty(n_out, dtype=np.float32)
        self.lib.oracle_f16_to_q8w(n_out, n_in, w.ctypes.data_as(C.POINTER(C.c_uint16)),
                                   wq.ctypes.data_as(C.POINTER(C.c_int8)), _fp(scales))
        return wq, scales

    def q8w_gemv(self, wq, scales, x):
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        scales = np.ascontiguousarray(scales, dtype=np.float32)
        xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
        n_out, n_in = wq.shape
        y = np.empty((xs.shape[0], n_out), dtype=np.float32)
        for m in range(xs.shape[0]):
            self.lib.oracle_q8w_gemv_m1(n_out, n_in, _fp(xs[m]),
                                        wq.ctypes.data_as(C.POINTER(C.c_int8)), _fp(scales), _fp(y[m]))
        return y[0] if np.ndim(x) == 1 else y

    def f16_linear_f64(self, w_f16, x):
        """cpu_scalar_w_quant_mN for F16 weights: [m, n_in] x [n_out, n_in] -> [m, n_out]."""
        w = np.ascontiguousarray(w_f16, dtype=np.uint16)
        xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
        n_out, n_in = w.shape
        y = np.empty((xs.shape[0], n_out), dtype=np.float32)
        self.lib.oracle_f16_linear_f64.argtypes = [C.c_size_t] * 3 + [c_float_p, C.POINTER(C.c_uint16),
                                                                      c_float_p]
        self.lib.oracle_f16_linear_f64(xs.shape[0], n_out, n_in, _fp(xs),
                                       w.ctypes.data_as(C.POINTER(C.c_uint16)), _fp(y))
        return y[0] if np.ndim(x) == 1 else y

    def rmsnorm(self, x, w, eps):
        xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
        w = np.ascontiguousarray(w, dtype=np.float32)
        y = np.empty_like(xs)
        self.lib.oracle_rmsnorm_rows(xs.shape[0], xs.shape[1], _fp(xs), _fp(w), eps, _fp(y))
        return y[0] if np.ndim(x) == 1 else y

    def spec_head_geometry(self, vocab, d_model, stride=0, topk=0):
        """(sketch_dim, topk) or None where the reference builds no sketch."""
        sd, k = C.c_size_t(), C.c_size_t()
        self.lib.oracle_spec_head_geometry.argtypes = [C.c_size_t] * 4 + [C.POINTER(C.c_size_t)] * 2
        if self.lib.oracle_spec_head_geometry(vocab, d_model, stride, topk, C.byref(sd), C.byref(k)):
            return None
        return sd.value, k.value

    def spec_head_build(self, w_f16, stride=0, topk=0):
        """The reference's sketch of a [vocab, d_model] binary16 table, or None."""
        return OracleSpecHead(self.lib, w_f16, stride, topk)._or_none()

    def softcap(self, row, cap):
        out = row.copy()
        self.lib.oracle_softcap_inplace(out.size, _fp(out), cap)
        return out

    def session(self, temperature=0.0, top_p=1.0, top_k=0, seed=0):
        s = SessionSampler()
        self.lib.oracle_session_defaults(C.byref(s))
        self.lib.oracle_session_apply_opts(C.byref(s), temperature, top_p, top_k, C.c_uint64(seed))
        return s

    def finalize_row(self, sess, row, softcap=0.0):
        tmp = row.copy()
        return int(self.lib.oracle_finalize_row(C.byref(sess), tmp.size, _fp(tmp), softcap))

    def finalize_batch(self, sess, rows, softcap=0.0):
        tmp = np.ascontiguousarray(rows, dtype=np.float32).copy()
        k, n = tmp.shape
        out = np.empty(k, dtype=np.int32)
        self.lib.oracle_finalize_batch(C.byref(sess), k, n, _fp(tmp), softcap, _ip(out))
        return out

    def spec_verify(self, target, q, draft, u, temperature):
        target = np.ascontiguousarray(target, dtype=np.float32)
        q = np.ascontiguousarray(q, dtype=np.float32)
        draft = np.ascontiguousarray(draft, dtype=np.int32)
        u = np.ascontiguousarray(u, dtype=np.float32)
        L = draft.size
        n = target.shape[1]
        assert target.shape[0] == L + 1 and q.shape == (L, n) and u.size == L + 1
        out = np.full(L + 1, -1, dtype=np.int32)
        nacc = self.lib.oracle_spec_verify(L, n, _fp(target), n, _fp(q), n, _ip(draft), _fp(u),
                                           temperature, _ip(out))
        return int(nacc), out

    def batch_chain_u(self, logits, u, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, hist=None,
                      hist_len=None, rep=1.0, freq=0.0, pres=0.0, threads=1):
        rows, n = logits.shape
        out = np.empty(rows, dtype=np.int32)
        prm = ChainParams(temperature, top_k, top_p, min_p)
        hp = _ip(hist) if hist is not None else None
        hl = _ip(hist_len) if hist_len is not None else None
        hld = hist.shape[1] if hist is not None else 0
        self.lib.oracle_batch_chain_u(rows, n, _fp(logits), n, C.byref(prm), hp, hld, hl, rep, freq,
                                      pres, _fp(u), _ip(out), threads)
        return out


# ---------------------------------------------------------------------------------------------
# The compiled reference (built from the reference's own sources by `make -C oracle ref`).
# ---------------------------------------------------------------------------------------------
class RefWorkspace(C.Structure):
    _fields_ = [("probs", c_float_p), ("n_vocab", C.c_size_t)]


def ref_path(fast=False):
    return os.path.join(ORACLE_DIR, "_ref",
                        "libgeist_ref_sampler_fast.so" if fast else "libgeist_ref_sampler.so")


def load_ref_f16gemv(fast=False):
    """The reference's f16_gemv_m1 compiled from its own sources, or None where not built. Loaded
    with lazy binding: the unit that defines fp16_to_fp32 also holds GGUF functions whose
    dependencies are not linked and are never called."""
    path = os.path.join(ORACLE_DIR, "_ref",
                        "libgeist_ref_f16gemv_fast.so" if fast else "libgeist_ref_f16gemv.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path, mode=os.RTLD_LAZY)
    lib.f16_gemv_m1.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.POINTER(C.c_uint16), c_float_p]
    lib.f16_gemv_m1.restype = None
    lib.fp16_to_fp32.restype = C.c_float
    lib.fp16_to_fp32.argtypes = [C.c_uint16]
    lib.f16_to_q8w.argtypes = [C.c_size_t, C.c_size_t, C.POINTER(C.c_uint16), C.POINTER(C.c_int8),
                               c_float_p]
    lib.f16_to_q8w.restype = None
    lib.q8w_gemv_m1.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.POINTER(C.c_int8), c_float_p,
                                c_float_p]
    lib.q8w_gemv_m1.restype = None
    return lib


def load_ref(fast=False):
    """Returns the compiled reference library, or None where it has not been built."""
    path = ref_path(fast)
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path)
    lib.geist_rng_next_u64.restype = C.c_uint64
    lib.geist_rng_next_unit.restype = C.c_float
    lib.geist_sampler_argmax.restype = C.c_int32
    lib.geist_sampler_argmax.argtypes = [C.c_size_t, c_float_p]
    lib.geist_sampler_temperature.restype = C.c_int32
    lib.geist_sampler_temperature.argtypes = [C.c_size_t, c_float_p, C.c_float,
                                              C.POINTER(OracleRng)]
    lib.geist_sampler_workspace_init.argtypes = [C.POINTER(RefWorkspace), C.c_size_t]
    lib.geist_sampler_workspace_destroy.argtypes = [C.POINTER(RefWorkspace)]
    lib.geist_sampler_top_k_ws.restype = C.c_int32
    lib.geist_sampler_top_k_ws.argtypes = [C.POINTER(RefWorkspace), c_float_p, C.c_int, C.c_float,
                                           C.POINTER(OracleRng)]
    lib.geist_sampler_top_p_ws.restype = C.c_int32
    lib.geist_sampler_top_p_ws.argtypes = [C.POINTER(RefWorkspace), c_float_p, C.c_float, C.c_float,
                                           C.POINTER(OracleRng)]
    return lib


class _SpecHeadStruct(C.Structure):
    _fields_ = [("vocab", C.c_size_t), ("d_model", C.c_size_t), ("sketch_dim", C.c_size_t),
                ("topk", C.c_size_t), ("dims", C.POINTER(C.c_uint32)),
                ("sketch", C.POINTER(C.c_int8)), ("row_scale", c_float_p),
                ("w_drop", c_float_p), ("w_l1", c_float_p)]


class OracleSpecHead:
    """oracle_spec_head_build / _try (oracle/spec_head_oracle.h)."""

    def __init__(self, lib, w_f16, stride=0, topk=0):
        self.lib = lib
        self.w = np.ascontiguousarray(w_f16, dtype=np.uint16)
        V, H = self.w.shape
        lib.oracle_spec_head_build.restype = C.POINTER(_SpecHeadStruct)
        lib.oracle_spec_head_build.argtypes = [C.POINTER(C.c_uint16)] + [C.c_size_t] * 4
        lib.oracle_spec_head_free.argtypes = [C.POINTER(_SpecHeadStruct)]
        lib.oracle_spec_head_free.restype = None
        lib.oracle_spec_head_try.argtypes = [C.POINTER(_SpecHeadStruct), C.POINTER(C.c_uint16),
                                             c_float_p, C.c_int, C.POINTER(C.c_int32), c_float_p,
                                             C.POINTER(C.c_size_t), c_float_p]
        self.p = lib.oracle_spec_head_build(self.w.ctypes.data_as(C.POINTER(C.c_uint16)), V, H,
                                            stride, topk)
        if self.p:
            st = self.p.contents
            self.sketch_dim, self.topk = st.sketch_dim, st.topk
            self.dims = np.ctypeslib.as_array(st.dims, (st.sketch_dim,)).copy()
            self.sketch = np.ctypeslib.as_array(st.sketch, (V, st.sketch_dim)).copy()
            self.row_scale = np.ctypeslib.as_array(st.row_scale, (V,)).copy()
            self.w_drop = np.ctypeslib.as_array(st.w_drop, (V,)).copy()
            self.w_l1 = np.ctypeslib.as_array(st.w_l1, (V,)).copy()

    def _or_none(self):
        return self if self.p else None

    def try_row(self, h, verify=False):
        """-> dict(token, certain, rough, n_finalists, cutoff)."""
        h = np.ascontiguousarray(h, dtype=np.float32)
        V = self.w.shape[0]
        rough = np.empty(V, dtype=np.float32)
        tok, nf, cut = C.c_int32(), C.c_size_t(), C.c_float()
        certain = self.lib.oracle_spec_head_try(self.p, self.w.ctypes.data_as(C.POINTER(C.c_uint16)),
                                                _fp(h), int(verify), C.byref(tok), _fp(rough),
                                                C.byref(nf), C.byref(cut))
        return dict(token=tok.value, certain=bool(certain), rough=rough, n_finalists=nf.value,
                    cutoff=cut.value)

    def __del__(self):
        if getattr(self, "p", None):
            self.lib.oracle_spec_head_free(self.p)
            self.p = None


# ---- Q6_K tables ---------------------------------------------------------------------------
Q6K_BLOCK_BYTES, Q6K_BLOCK_ELEMS = 210, 256


def random_q6k_table(g, n_out, n_in, scale_mode="mixed"):
    """A [n_out, n_in] table of Q6_K super-blocks as uint8 [n_out, n_in / 256 * 210]: every bit
    pattern of ql / qh, int8 scales over their whole range (with 0, 127 and -128 forced in),
    binary16 super-block scales that are normal, subnormal, zero or negative (never inf / NaN)."""
    assert n_in % Q6K_BLOCK_ELEMS == 0
    nb = n_in // Q6K_BLOCK_ELEMS
    t = g.integers(0, 256, (n_out, nb, Q6K_BLOCK_BYTES), dtype=np.uint8)
    sc = g.integers(-128, 128, (n_out, nb, 16)).astype(np.int8)
    if scale_mode == "mixed":
        sc[g.random((n_out, nb, 16)) < 0.05] = 0
        sc[g.random((n_out, nb, 16)) < 0.02] = 127
        sc[g.random((n_out, nb, 16)) < 0.02] = -128
    t[:, :, 192:208] = sc.view(np.uint8)
    d = (g.standard_normal((n_out, nb)) * 0.01).astype(np.float16)
    kind = g.random((n_out, nb))
    d[kind < 0.03] = np.float16(0.0)
    d = d.view(np.uint16).copy()
    sub = (kind >= 0.03) & (kind < 0.08)           # subnormal: exponent bits 0, mantissa random
    d[sub] = (g.integers(1, 1024, int(sub.sum())) | (g.integers(0, 2, int(sub.sum())) << 15)).astype(np.uint16)
    t[:, :, 208] = (d & 0xFF).astype(np.uint8)
    t[:, :, 209] = (d >> 8).astype(np.uint8)
    return np.ascontiguousarray(t.reshape(n_out, nb * Q6K_BLOCK_BYTES))


def oracle_q6k_linear(lib, w_q6k, x, n_in):
    """(float) sum_k (double) x[i][k] * (double) dequant(w[j][k]) for every activation row."""
    xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    n_out = w_q6k.shape[0]
    y = np.empty((xs.shape[0], n_out), dtype=np.float32)
    lib.oracle_q6k_linear_f64.argtypes = [C.c_size_t] * 3 + [c_float_p, C.c_void_p, c_float_p]
    lib.oracle_q6k_linear_f64.restype = None
    lib.oracle_q6k_linear_f64(xs.shape[0], n_out, n_in, _fp(xs), w_q6k.ctypes.data_as(C.c_void_p),
                              _fp(y))
    return y


def oracle_q6k_gemv_x86(lib, w_q6k, x, n_in):
    """oracle_q6k_gemv_x86: the x86 backend's one-row decode kernel over a Q6_K table."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    n_out = w_q6k.shape[0]
    y = np.full(n_out, np.nan, dtype=np.float32)
    lib.oracle_q6k_gemv_x86.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_void_p, c_float_p]
    lib.oracle_q6k_gemv_x86.restype = C.c_int
    rc = lib.oracle_q6k_gemv_x86(n_out, n_in, _fp(x), w_q6k.ctypes.data_as(C.c_void_p), _fp(y))
    assert rc == 0
    return y


def oracle_q8k_quantize(lib, x):
    """(d [n_super], qs int8 [n_in], bsums int16 [n_in / 16]) of one activation row."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    ns = x.size // 256
    d = np.empty(ns, dtype=np.float32)
    qs = np.empty(ns * 256, dtype=np.int8)
    bs = np.empty(ns * 16, dtype=np.int16)
    lib.oracle_q8k_quantize.argtypes = [C.c_size_t, c_float_p, c_float_p, C.c_void_p, C.c_void_p]
    lib.oracle_q8k_quantize.restype = None
    lib.oracle_q8k_quantize(ns, _fp(x), _fp(d), qs.ctypes.data_as(C.c_void_p),
                            bs.ctypes.data_as(C.c_void_p))
    return d, qs, bs


def load_ref_q6kgemv(fast=False):
    """The reference's q6k_gemv_m1 compiled from its tree, or None where not built."""
    path = os.path.join(ORACLE_DIR, "_ref",
                        "libgeist_ref_q6kgemv_fast.so" if fast else "libgeist_ref_q6kgemv.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path, mode=os.RTLD_LAZY)
    lib.q6k_gemv_m1.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_void_p, c_float_p]
    lib.q6k_gemv_m1.restype = None
    return lib


def ref_q6k_gemv_m1(ref, w_q6k, x, n_in):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    n_out = w_q6k.shape[0]
    y = np.full(n_out, np.nan, dtype=np.float32)
    ref.q6k_gemv_m1(n_out, n_in, _fp(x), w_q6k.ctypes.data_as(C.c_void_p), _fp(y))
    return y


def oracle_dequant_q6k(lib, w_q6k, n_in):
    out = np.empty((w_q6k.shape[0], n_in), dtype=np.float32)
    lib.oracle_dequant_q6_K_row.argtypes = [C.c_void_p, c_float_p, C.c_size_t]
    lib.oracle_dequant_q6_K_row.restype = None
    for j in range(w_q6k.shape[0]):
        lib.oracle_dequant_q6_K_row(w_q6k[j].ctypes.data_as(C.c_void_p), _fp(out[j]), n_in)
    return out


def load_ref_wquant(fast=False):
    """The reference's portable linear kernels compiled from its tree, or None where not built
    (lazy binding, as for load_ref_f16gemv)."""
    path = os.path.join(ORACLE_DIR, "_ref",
                        "libgeist_ref_wquant_fast.so" if fast else "libgeist_ref_wquant.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path, mode=os.RTLD_LAZY)
    lib.ref_wquant_linear.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, c_float_p, C.c_size_t,
                                      c_float_p]
    lib.dequant_q6_K_row.argtypes = [C.c_void_p, c_float_p, C.c_size_t]
    lib.dequant_q6_K_row.restype = None
    lib.dequant_q4_K_row.argtypes = [C.c_void_p, c_float_p, C.c_size_t]
    lib.dequant_q4_K_row.restype = None
    return lib


def ref_f16_linear(ref, w_f16_bits, x):
    """cpu_scalar_w_quant_m1 / _mN over an F16 table (uint16 bit patterns [n_out, n_in]), compiled
    from the reference's tree."""
    xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    w = np.ascontiguousarray(w_f16_bits, dtype=np.uint16)
    n_out, n_in = w.shape
    y = np.full((xs.shape[0], n_out), np.nan, dtype=np.float32)
    rc = ref.ref_wquant_linear(ref.ref_dtype_f16(), w.ctypes.data_as(C.c_void_p), n_out, n_in,
                               _fp(xs), xs.shape[0], _fp(y))
    assert rc == 0
    return y


def ref_q6k_linear(ref, w_q6k, x, n_in):
    xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    n_out = w_q6k.shape[0]
    y = np.full((xs.shape[0], n_out), np.nan, dtype=np.float32)
    rc = ref.ref_wquant_linear(ref.ref_dtype_q6_K(), w_q6k.ctypes.data_as(C.c_void_p), n_out, n_in,
                               _fp(xs), xs.shape[0], _fp(y))
    assert rc == 0
    return y


# ---- Q4_K tables ---------------------------------------------------------------------------
Q4K_BLOCK_BYTES, Q4K_BLOCK_ELEMS = 144, 256


def _random_f16_scales(g, shape, sigma):
    """binary16 values that are normal, subnormal, zero or negative, never inf / NaN, as uint16."""
    d = (g.standard_normal(shape) * sigma).astype(np.float16)
    kind = g.random(shape)
    d[kind < 0.03] = np.float16(0.0)
    d = d.view(np.uint16).copy()
    sub = (kind >= 0.03) & (kind < 0.08)
    d[sub] = (g.integers(1, 1024, int(sub.sum())) | (g.integers(0, 2, int(sub.sum())) << 15)).astype(np.uint16)
    return d


def random_q4k_table(g, n_out, n_in):
    """A [n_out, n_in] table of Q4_K super-blocks as uint8 [n_out, n_in / 256 * 144]: every bit
    pattern of the packed scales / minima and of the 4-bit values, binary16 d and dmin of either
    sign and of very different magnitudes (so that d * sc * q - dmin * m does round)."""
    assert n_in % Q4K_BLOCK_ELEMS == 0
    nb = n_in // Q4K_BLOCK_ELEMS
    t = g.integers(0, 256, (n_out, nb, Q4K_BLOCK_BYTES), dtype=np.uint8)
    d = _random_f16_scales(g, (n_out, nb), 0.01)
    dmin = _random_f16_scales(g, (n_out, nb), 0.01)
    big = g.random((n_out, nb)) < 0.3      # dmin a few thousand times d: the subtraction rounds
    dmin[big] = (g.standard_normal(int(big.sum())) * 8.0).astype(np.float16).view(np.uint16)
    t[:, :, 0] = (d & 0xFF).astype(np.uint8)
    t[:, :, 1] = (d >> 8).astype(np.uint8)
    t[:, :, 2] = (dmin & 0xFF).astype(np.uint8)
    t[:, :, 3] = (dmin >> 8).astype(np.uint8)
    return np.ascontiguousarray(t.reshape(n_out, nb * Q4K_BLOCK_BYTES))


def oracle_q4k_linear(lib, w_q4k, x, n_in):
    xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    n_out = w_q4k.shape[0]
    y = np.empty((xs.shape[0], n_out), dtype=np.float32)
    lib.oracle_q4k_linear_f64.argtypes = [C.c_size_t] * 3 + [c_float_p, C.c_void_p, c_float_p]
    lib.oracle_q4k_linear_f64.restype = None
    lib.oracle_q4k_linear_f64(xs.shape[0], n_out, n_in, _fp(xs), w_q4k.ctypes.data_as(C.c_void_p),
                              _fp(y))
    return y


def oracle_dequant_q4k(lib, w_q4k, n_in):
    out = np.empty((w_q4k.shape[0], n_in), dtype=np.float32)
    lib.oracle_dequant_q4_K_row.argtypes = [C.c_void_p, c_float_p, C.c_size_t]
    lib.oracle_dequant_q4_K_row.restype = None
    for j in range(w_q4k.shape[0]):
        lib.oracle_dequant_q4_K_row(w_q4k[j].ctypes.data_as(C.c_void_p), _fp(out[j]), n_in)
    return out


def ref_q4k_linear(ref, w_q4k, x, n_in):
    xs = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    n_out = w_q4k.shape[0]
    y = np.full((xs.shape[0], n_out), np.nan, dtype=np.float32)
    rc = ref.ref_wquant_linear(ref.ref_dtype_q4_K(), w_q4k.ctypes.data_as(C.c_void_p), n_out, n_in,
                               _fp(xs), xs.shape[0], _fp(y))
    assert rc == 0
    return y


def oracle_q4k_gemv_x86(lib, w_q4k, x, n_in):
    """oracle_q4k_gemv_x86: the x86 backend's one-row decode kernel over a Q4_K table."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    n_out = w_q4k.shape[0]
    y = np.full(n_out, np.nan, dtype=np.float32)
    lib.oracle_q4k_gemv_x86.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_void_p, c_float_p]
    lib.oracle_q4k_gemv_x86.restype = C.c_int
    rc = lib.oracle_q4k_gemv_x86(n_out, n_in, _fp(x), w_q4k.ctypes.data_as(C.c_void_p), _fp(y))
    assert rc == 0, rc
    return y


def oracle_q8k_row_quantize(lib, x):
    """(d, qs int8 [n_in], bsums int16 [n_in / 16]) of one activation row, one scale per row."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    ns = x.size // 256
    d = np.empty(1, dtype=np.float32)
    qs = np.empty(ns * 256, dtype=np.int8)
    bs = np.empty(ns * 16, dtype=np.int16)
    lib.oracle_q8k_row_quantize.argtypes = [C.c_size_t, c_float_p, c_float_p, C.c_void_p, C.c_void_p]
    lib.oracle_q8k_row_quantize.restype = None
    lib.oracle_q8k_row_quantize(ns, _fp(x), _fp(d), qs.ctypes.data_as(C.c_void_p),
                                bs.ctypes.data_as(C.c_void_p))
    return float(d[0]), qs, bs


def load_ref_q6kmn():
    """The reference's int8 copy of a Q6_K table (q6k_to_w8a8_row, w8x8 / w8x16_repack), its
    activation quantiser and its W8A8 kernels compiled from its tree (strict flags), or None where
    not built."""
    path = os.path.join(ORACLE_DIR, "_ref", "libgeist_ref_q6kmn.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path, mode=os.RTLD_LAZY)
    vp, sz = C.c_void_p, C.c_size_t
    lib.q6k_to_w8a8_row.argtypes = [sz, vp, vp, vp, vp]
    lib.q6k_to_w8a8_row.restype = None
    lib.w4a8_quantize_acts_row.argtypes = [sz, c_float_p, vp, vp]
    lib.w4a8_quantize_acts_row.restype = C.c_float
    lib.w8a8_isa_is_vnni.restype = C.c_int
    for name in ("w8x8_repack", "w8x16_repack"):
        getattr(lib, name).argtypes = [sz, sz, vp, vp, vp, vp, vp, vp]
        getattr(lib, name).restype = None
    for name in ("w8a8_gemm", "w8x8_gemm", "w8x16_gemm"):
        getattr(lib, name).argtypes = [sz, sz, sz, vp, vp, vp, vp, vp, vp, c_float_p]
        getattr(lib, name).restype = None
    return lib


def ref_q6k_mN_prepare(ref, w_q6k, n_in):
    """cpu_x86_linear_q6k_resolve (linear_q6k.c:84-156) by the reference's own calls: the int8 copy
    row by row, interleaved in eights or sixteens on a VNNI host. Returns run(x) -> (y, lanes),
    which is cpu_x86_linear_q6k_mN (:234-300): w4a8_quantize_acts_row per row, the sums again per
    sixteen, then the kernel the host and the table's row count select."""
    n_out, nblk = w_q6k.shape[0], n_in // 16
    w = np.ascontiguousarray(w_q6k)
    row_bytes = n_in // 256 * 210
    vp = lambda a: a.ctypes.data_as(C.c_void_p)  # noqa: E731
    wq = np.zeros((n_out, n_in), dtype=np.uint8)
    ws = np.zeros((n_out, nblk), dtype=np.float32)
    wo = np.zeros((n_out, nblk), dtype=np.float32)
    for r in range(n_out):
        ref.q6k_to_w8a8_row(n_in, C.c_void_p(w.ctypes.data + r * row_bytes),
                            C.c_void_p(wq.ctypes.data + r * n_in),
                            C.c_void_p(ws.ctypes.data + r * nblk * 4),
                            C.c_void_p(wo.ctypes.data + r * nblk * 4))
    lanes = bool(ref.w8a8_isa_is_vnni()) and n_out % 8 == 0
    which = "w8x16" if n_out % 16 == 0 else "w8x8"
    if lanes:
        il_q, il_s, il_o = np.zeros_like(wq), np.zeros_like(ws), np.zeros_like(wo)
        getattr(ref, which + "_repack")(n_out, n_in, vp(wq), vp(ws), vp(wo), vp(il_q), vp(il_s), vp(il_o))

    def run(x):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, n_in)
        m = x.shape[0]
        acts = np.zeros((m, n_in), dtype=np.int8)
        sum_a = np.zeros((m, nblk), dtype=np.int32)
        scale_x = np.zeros(m, dtype=np.float32)
        for j in range(m):
            scale_x[j] = ref.w4a8_quantize_acts_row(n_in, _fp(x[j]),
                                                    C.c_void_p(acts.ctypes.data + j * n_in),
                                                    C.c_void_p(sum_a.ctypes.data + j * nblk * 4))
            # linear_q6k.c:271-279: the sums again at the W8A8 granularity of sixteen
            sum_a[j] = acts[j].reshape(nblk, 16).astype(np.int32).sum(axis=1)
        y = np.full((m, n_out), np.nan, dtype=np.float32)
        if lanes:
            getattr(ref, which + "_gemm")(m, n_out, nblk, vp(il_q), vp(il_s), vp(il_o), vp(acts),
                                          vp(sum_a), vp(scale_x), _fp(y))
        else:
            ref.w8a8_gemm(m, n_out, nblk, vp(wq), vp(ws), vp(wo), vp(acts), vp(sum_a), vp(scale_x),
                          _fp(y))
        return y, lanes

    return run


def ref_q6k_linear_mN(ref, w_q6k, x, n_in):
    """(y, lanes) of the reference's load-time copy and batch projection, see ref_q6k_mN_prepare."""
    return ref_q6k_mN_prepare(ref, w_q6k, n_in)(x)


def oracle_q8_sym_row_quantize(lib, x):
    """(scale, q int8 [n], sums int32 [n / 16]) of one row as quantize_x_int8_sym leaves it."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    d = np.empty(1, dtype=np.float32)
    q = np.empty(x.size, dtype=np.int8)
    sm = np.empty(x.size // 16, dtype=np.int32)
    lib.oracle_q8_sym_row_quantize.argtypes = [C.c_size_t, c_float_p, c_float_p, C.c_void_p, C.c_void_p]
    lib.oracle_q8_sym_row_quantize.restype = None
    lib.oracle_q8_sym_row_quantize(x.size, _fp(x), _fp(d), q.ctypes.data_as(C.c_void_p),
                                   sm.ctypes.data_as(C.c_void_p))
    return float(d[0]), q, sm


def oracle_q6k_linear_x86(lib, w_q6k, x, n_in, vnni=True):
    """oracle_q6k_linear_x86: the x86 backend's projection of a batch over a Q6_K table."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, n_in)
    m, n_out = x.shape[0], w_q6k.shape[0]
    y = np.full((m, n_out), np.nan, dtype=np.float32)
    lib.oracle_q6k_linear_x86.argtypes = [C.c_size_t, C.c_size_t, C.c_size_t, c_float_p,
                                          C.c_void_p, c_float_p, C.c_int]
    lib.oracle_q6k_linear_x86.restype = C.c_int
    rc = lib.oracle_q6k_linear_x86(m, n_out, n_in, _fp(x), w_q6k.ctypes.data_as(C.c_void_p), _fp(y),
                                   1 if vnni else 0)
    assert rc == 0, rc
    return y


def oracle_q8kx4_row_quantize(lib, x):
    """(d, qs int8 [n_in], bsums int16 [n_in / 16]) of one row as quantize_q8_Kx4 leaves it."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    ns = x.size // 256
    d = np.empty(1, dtype=np.float32)
    qs = np.empty(ns * 256, dtype=np.int8)
    bs = np.empty(ns * 16, dtype=np.int16)
    lib.oracle_q8kx4_row_quantize.argtypes = [C.c_size_t, c_float_p, c_float_p, C.c_void_p,
                                              C.c_void_p]
    lib.oracle_q8kx4_row_quantize.restype = None
    lib.oracle_q8kx4_row_quantize(ns, _fp(x), _fp(d), qs.ctypes.data_as(C.c_void_p),
                                  bs.ctypes.data_as(C.c_void_p))
    return float(d[0]), qs, bs


def oracle_q4k_linear_x86(lib, w_q4k, x, n_in, avx512=True):
    """oracle_q4k_linear_x86: the x86 backend's projection of a batch over a Q4_K table."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, n_in)
    m, n_out = x.shape[0], w_q4k.shape[0]
    y = np.full((m, n_out), np.nan, dtype=np.float32)
    lib.oracle_q4k_linear_x86.argtypes = [C.c_size_t, C.c_size_t, C.c_size_t, c_float_p,
                                          C.c_void_p, c_float_p, C.c_int]
    lib.oracle_q4k_linear_x86.restype = C.c_int
    rc = lib.oracle_q4k_linear_x86(m, n_out, n_in, _fp(x), w_q4k.ctypes.data_as(C.c_void_p), _fp(y),
                                   1 if avx512 else 0)
    assert rc == 0, rc
    return y


Q4KX8_BLOCK_BYTES = 1152
Q8KX4_BLOCK_BYTES = 1168     # struct block_q8_Kx4: d[4] float, qs[1024] int8, bsums[64] int16


def load_ref_q4kgemv(fast=False):
    """The reference's q4k_to_q4kx8_matrix and q4kx8_gemv_m1 compiled from its tree, or None where
    not built."""
    path = os.path.join(ORACLE_DIR, "_ref",
                        "libgeist_ref_q4kgemv_fast.so" if fast else "libgeist_ref_q4kgemv.so")
    if not os.path.exists(path):
        return None
    lib = C.CDLL(path, mode=os.RTLD_LAZY)
    lib.q4k_to_q4kx8_matrix.argtypes = [C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p]
    lib.q4k_to_q4kx8_matrix.restype = None
    lib.q4kx8_gemv_m1.argtypes = [C.c_size_t, C.c_size_t, c_float_p, C.c_void_p, c_float_p]
    lib.q4kx8_gemv_m1.restype = None
    lib.quantize_q8_Kx4.argtypes = [C.c_size_t, c_float_p, C.c_void_p]
    lib.quantize_q8_Kx4.restype = None
    lib.q4kx8_gemm_avx512.argtypes = [C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p,
                                      c_float_p]
    lib.q4kx8_gemm_avx512.restype = None
    return lib


def ref_q4k_gemv_m1(ref, w_q4k, x, n_in):
    """The table interleaved by the reference's repacker, then its decode kernel."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    n_out = w_q4k.shape[0]
    assert n_out % 8 == 0 and n_in % 256 == 0
    blob = np.zeros(n_out // 8 * (n_in // 256) * Q4KX8_BLOCK_BYTES + 64, dtype=np.uint8)
    w = np.ascontiguousarray(w_q4k)
    ref.q4k_to_q4kx8_matrix(n_in, n_out, w.ctypes.data_as(C.c_void_p), blob.ctypes.data_as(C.c_void_p))
    y = np.full(n_out, np.nan, dtype=np.float32)
    ref.q4kx8_gemv_m1(n_out, n_in, _fp(x), blob.ctypes.data_as(C.c_void_p), _fp(y))
    return y


def ref_q4k_linear_mN(ref, w_q4k, x, n_in):
    """The reference's calls in the order of cpu_x86_linear_q4k_mN (linear_q4k.c:198-250): a row
    count that is no multiple of 4 runs the decode kernel row by row; otherwise quantize_q8_Kx4 per
    four rows, then q4kx8_gemm_avx512 over the interleaved table."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, n_in)
    m, n_out, ns = x.shape[0], w_q4k.shape[0], n_in // 256
    assert n_out % 8 == 0 and n_in % 256 == 0
    if m % 4 != 0:
        return np.stack([ref_q4k_gemv_m1(ref, w_q4k, x[i], n_in) for i in range(m)])
    blob = np.zeros(n_out // 8 * ns * Q4KX8_BLOCK_BYTES + 64, dtype=np.uint8)
    w = np.ascontiguousarray(w_q4k)
    ref.q4k_to_q4kx8_matrix(n_in, n_out, w.ctypes.data_as(C.c_void_p), blob.ctypes.data_as(C.c_void_p))
    acts = np.zeros(m // 4 * ns * Q8KX4_BLOCK_BYTES + 64, dtype=np.uint8)
    for mt in range(m // 4):
        ref.quantize_q8_Kx4(n_in, _fp(x[4 * mt:4 * mt + 4]),
                            C.c_void_p(acts.ctypes.data + mt * ns * Q8KX4_BLOCK_BYTES))
    y = np.full((m, n_out), np.nan, dtype=np.float32)
    ref.q4kx8_gemm_avx512(m, n_out, n_in, acts.ctypes.data_as(C.c_void_p),
                          blob.ctypes.data_as(C.c_void_p), _fp(y))
    return y
