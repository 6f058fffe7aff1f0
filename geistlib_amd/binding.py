"""ctypes binding of include/geist_sampler_hip.h. Device memory comes from torch tensors
(`tensor.data_ptr()`); nothing here computes on logits."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))

GEIST_HIP_OK = 0
PRECEDENCE_REFERENCE = 0
PRECEDENCE_CHAIN = 1

_STATUS = {0: "OK", 1: "E_OOM", 2: "E_INVALID_ARG", 3: "E_INTERNAL", 7: "E_UNSUPPORTED",
           9: "E_BACKEND"}


class GeistHipError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"{_STATUS.get(code, code)}: {text}")
        self.code = code


class Rows(C.Structure):
    _fields_ = [("d_logits", C.c_void_p), ("ld", C.c_size_t), ("rows", C.c_size_t),
                ("n_vocab", C.c_size_t), ("d_history", C.c_void_p), ("history_ld", C.c_size_t),
                ("d_history_len", C.c_void_p), ("d_allowed", C.c_void_p),
                ("allowed_ld", C.c_size_t)]


class SampleParams(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("top_k", C.c_int),
                ("min_p", C.c_float), ("repetition_penalty", C.c_float),
                ("frequency_penalty", C.c_float), ("presence_penalty", C.c_float),
                ("logit_softcap", C.c_float), ("precedence", C.c_int)]

    @classmethod
    def make(cls, temperature=0.0, top_p=1.0, top_k=0, min_p=0.0, rep=1.0, freq=0.0, pres=0.0,
             softcap=0.0, precedence=PRECEDENCE_CHAIN):
        return cls(temperature, top_p, top_k, min_p, rep, freq, pres, softcap, precedence)


class SpecResult(C.Structure):
    """struct geist_hip_spec_result."""
    _fields_ = [("token", C.c_int32), ("answered", C.c_int32), ("n_finalists", C.c_int32),
                ("n_listed", C.c_int32), ("cutoff", C.c_float), ("best_exact", C.c_float)]


class SpecHeadView(C.Structure):
    """struct geist_hip_spec_head_view."""
    _fields_ = [("n_vocab", C.c_size_t), ("d_model", C.c_size_t), ("sketch_dim", C.c_size_t),
                ("topk", C.c_size_t), ("d_dims", C.c_void_p), ("d_sketch", C.c_void_p),
                ("d_row_scale", C.c_void_p), ("d_w_drop", C.c_void_p), ("d_w_l1", C.c_void_p),
                ("d_rough", C.c_void_p)]


def library_path(name="libgeist_sampler_hip.so"):
    """Where the built library lies; GEIST_HIP_LIB_DIR names another directory (an instrumented
    build, `make -C geistlib_amd phase-stamps`)."""
    return os.path.join(os.environ.get("GEIST_HIP_LIB_DIR") or os.path.join(HERE, "lib"), name)


_LIB = None


def load_library():
    """Loads the built HIP library. There is no fallback: a missing library is an error."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `make -C geistlib_amd` "
                           "(or __graft_entry__.build()); the sampling path has no CPU fallback")
    lib = C.CDLL(path)
    vp, sz, i32, f32 = C.c_void_p, C.c_size_t, C.c_int, C.c_float
    lib.geist_hip_sampler_create.argtypes = [i32, sz, sz, vp, C.POINTER(vp)]
    lib.geist_hip_sampler_destroy.argtypes = [vp]
    lib.geist_hip_sampler_destroy.restype = None
    lib.geist_hip_sampler_last_error.argtypes = [vp]
    lib.geist_hip_sampler_last_error.restype = C.c_char_p
    lib.geist_hip_sampler_sync.argtypes = [vp]
    lib.geist_hip_sampler_set_stream.argtypes = [vp, vp]
    lib.geist_hip_sampler_set_logits_hint.argtypes = [vp, i32]
    lib.geist_hip_sampler_set_projection.argtypes = [vp, i32]
    lib.geist_hip_sampler_prepare.argtypes = [vp, C.POINTER(SampleParams), sz]
    lib.geist_hip_sampler_set_wait_limit.argtypes = [vp, C.c_uint32]
    lib.geist_hip_sampler_one_launch_topk.argtypes = [vp, i32]
    lib.geist_hip_sampler_one_launch_spec.argtypes = [vp, i32]
    lib.geist_hip_sampler_handoff_scope.argtypes = [vp, i32]
    lib.geist_hip_sampler_set_whole_row_walk.argtypes = [vp, i32]
    lib.geist_hip_sampler_notify_ids.argtypes = [vp, i32]
    lib.geist_hip_sampler_wait_ids.argtypes = [vp]
    lib.geist_hip_sampler_set_sums.argtypes = [vp, i32]
    lib.geist_hip_sampler_set_wait_spin.argtypes = [vp, C.c_uint32]
    lib.geist_hip_sample_rows.argtypes = [vp, C.POINTER(Rows), C.POINTER(SampleParams), vp, vp]
    lib.geist_hip_sample_rows_rng.argtypes = [vp, C.POINTER(Rows), C.POINTER(SampleParams), vp, i32,
                                              vp]
    lib.geist_hip_sample_rows_static.argtypes = [i32, vp, C.POINTER(Rows), C.POINTER(SampleParams),
                                                 vp, vp, C.c_char_p, sz]
    lib.geist_hip_argmax_f32.argtypes = [vp, vp, sz, C.POINTER(C.c_int32)]
    lib.geist_hip_apply_penalties.argtypes = [vp, vp, sz, sz, sz, vp, sz, vp, f32, f32, f32]
    lib.geist_hip_softmax_rows.argtypes = [vp, C.POINTER(Rows), C.POINTER(SampleParams), vp, sz]
    lib.geist_hip_spec_verify.argtypes = [vp, vp, sz, vp, sz, vp, vp, sz, sz, sz, f32, f32, vp, vp]
    lib.geist_hip_rng_draw_units.argtypes = [vp, vp, sz, vp]
    lib.geist_hip_malloc.argtypes = [vp, sz, C.POINTER(vp)]
    lib.geist_hip_free.argtypes = [vp, vp]
    lib.geist_hip_upload.argtypes = [vp, vp, vp, sz]
    lib.geist_hip_download.argtypes = [vp, vp, vp, sz]
    lib.geist_hip_host_malloc.argtypes = [vp, sz, C.POINTER(vp)]
    lib.geist_hip_host_free.argtypes = [vp, vp]
    lib.geist_hip_sampler_row_paths.argtypes = [vp, vp, sz]
    lib.geist_hip_sampler_topk_paths.argtypes = [vp, vp, sz]
    lib.geist_hip_logprob_rows.argtypes = [vp, vp, sz, sz, sz, f32, vp, sz, sz, vp, sz]
    lib.geist_hip_propose_drafts_ngram.argtypes = [vp, vp, sz, vp, vp, sz, sz, sz, vp, sz, vp, vp]
    lib.geist_hip_rmsnorm_rows.argtypes = [vp, vp, sz, vp, f32, sz, sz, vp, sz]
    lib.geist_hip_f16_gemv_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_f16_linear_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q6k_linear_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q6k_linear_reserve.argtypes = [vp, sz, sz]
    lib.geist_hip_q6k_packed_bytes.argtypes = [sz, sz]
    lib.geist_hip_q6k_packed_bytes.restype = sz
    lib.geist_hip_q6k_pack.argtypes = [vp, vp, sz, sz, vp]
    lib.geist_hip_q6k_packed_linear_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q6k_packed_gemv_x86_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q6k_gemv_x86_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q4k_packed_gemv_x86_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q4k_packed_linear_x86_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q6k_packed_linear_x86_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q6k_linear_x86_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_q8k_act_bytes.argtypes = [sz, sz]
    lib.geist_hip_q8k_act_bytes.restype = sz
    lib.geist_hip_q8k_quantize_rows.argtypes = [vp, vp, sz, sz, sz, vp]
    lib.geist_hip_q6k_packed_gemv_q8k.argtypes = [vp, vp, sz, sz, vp, vp]
    lib.geist_hip_q8k_row_act_bytes.argtypes = [sz]
    lib.geist_hip_q8k_row_act_bytes.restype = sz
    lib.geist_hip_q8k_row_quantize.argtypes = [vp, vp, sz, vp]
    lib.geist_hip_q4k_packed_gemv_q8k.argtypes = [vp, vp, sz, sz, vp, vp]
    lib.geist_hip_project_sample_rows_q6k_packed.argtypes = [vp, vp, sz, sz, sz, vp, f32, vp, sz,
                                                             vp, vp, sz, C.POINTER(SampleParams),
                                                             vp, vp, i32, vp]
    lib.geist_hip_q4k_packed_bytes.argtypes = [sz, sz]
    lib.geist_hip_q4k_packed_bytes.restype = sz
    lib.geist_hip_q4k_pack.argtypes = [vp, vp, sz, sz, vp]
    lib.geist_hip_q4k_packed_linear_rows.argtypes = [vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_project_sample_rows_q4k_packed.argtypes = [vp, vp, sz, sz, sz, vp, f32, vp, sz,
                                                             vp, vp, sz, C.POINTER(SampleParams),
                                                             vp, vp, i32, vp]
    lib.geist_hip_f16_to_q8w.argtypes = [vp, vp, sz, sz, vp, vp]
    lib.geist_hip_q8w_gemv_rows.argtypes = [vp, vp, vp, sz, sz, vp, sz, sz, vp, sz]
    lib.geist_hip_project_sample_rows.argtypes = [vp, vp, sz, sz, sz, vp, f32, vp, sz, vp, vp, sz,
                                                  C.POINTER(SampleParams), vp, vp, i32, vp]
    lib.geist_hip_project_sample_rows_q8w.argtypes = [vp, vp, sz, sz, sz, vp, f32, vp, vp, sz, vp,
                                                      vp, sz, C.POINTER(SampleParams), vp, vp,
                                                      i32, vp]
    lib.geist_hip_project_sample_rows_q6k.argtypes = [vp, vp, sz, sz, sz, vp, f32, vp, sz, vp, vp,
                                                      sz, C.POINTER(SampleParams), vp, vp, i32, vp]
    lib.geist_hip_spec_head_geometry.argtypes = [sz, sz, sz, sz, C.POINTER(sz), C.POINTER(sz)]
    lib.geist_hip_spec_head_build.argtypes = [vp, vp, sz, sz, sz, sz, C.POINTER(vp)]
    lib.geist_hip_spec_head_destroy.argtypes = [vp, vp]
    lib.geist_hip_spec_head_destroy.restype = None
    lib.geist_hip_spec_head_view.argtypes = [vp, C.POINTER(SpecHeadView)]
    lib.geist_hip_spec_head_try.argtypes = [vp, vp, vp, i32, vp]
    lib.geist_hip_spec_head_try_hidden.argtypes = [vp, vp, vp, vp, f32, vp, i32, vp]
    _LIB = lib
    return lib


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


class HostBuffer:
    """Page-locked host memory that the device addresses in place (geist_hip_host_malloc): pass it
    where a device tensor is expected (it has data_ptr()), read or write it through view()."""

    def __init__(self, sampler, nbytes):
        self.sampler, self.nbytes = sampler, int(nbytes)
        p = C.c_void_p()
        sampler._check(sampler.lib.geist_hip_host_malloc(sampler.h, self.nbytes, C.byref(p)))
        self.p = p

    def data_ptr(self):
        return self.p.value

    def view(self, dtype):
        import numpy as np
        dtype = np.dtype(dtype)
        buf = (C.c_char * self.nbytes).from_address(self.p.value)
        return np.frombuffer(buf, dtype=dtype, count=self.nbytes // dtype.itemsize)

    def close(self):
        if self.p and self.sampler.h:
            self.sampler.lib.geist_hip_host_free(self.sampler.h, self.p)
        self.p = C.c_void_p()


def sample_rows_static(rows, params, uniforms, out, device=0, stream=None):
    """geist_hip_sample_rows_static: sampling without a sampler object and without any
    allocation (the workspace is an array inside the library)."""
    lib = load_library()
    err = C.create_string_buffer(512)
    rc = lib.geist_hip_sample_rows_static(device, stream, C.byref(rows), C.byref(params),
                                          _ptr(uniforms), _ptr(out), err, len(err))
    if rc != GEIST_HIP_OK:
        raise GeistHipError(rc, err.value.decode())


class HipSampler:
    """One device workspace + stream, as one sampler workspace per session in the reference."""

    def __init__(self, max_rows, max_vocab, device=0, stream=None):
        self.lib = load_library()
        self.h = C.c_void_p()
        rc = self.lib.geist_hip_sampler_create(device, max_rows, max_vocab, stream, C.byref(self.h))
        if rc != GEIST_HIP_OK:
            raise GeistHipError(rc, "geist_hip_sampler_create failed")

    def close(self):
        if self.h:
            self.lib.geist_hip_sampler_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc != GEIST_HIP_OK:
            raise GeistHipError(rc, self.lib.geist_hip_sampler_last_error(self.h).decode())

    def set_wait_limit(self, polls):
        self._check(self.lib.geist_hip_sampler_set_wait_limit(self.h, C.c_uint32(polls)))

    def set_whole_row_walk(self, mode):
        """0 adaptive (default), 1 always spread over the row's chunks, 2 one workgroup."""
        self._check(self.lib.geist_hip_sampler_set_whole_row_walk(self.h, int(mode)))

    def one_launch_topk(self, enable=True):
        """Whether the top-k candidate path runs as one launch for batches that qualify."""
        rc = self.lib.geist_hip_sampler_one_launch_topk(self.h, 1 if enable else 0)
        if rc < 0:
            self._check(rc)
        return bool(rc)

    def handoff_scope(self, always_agent=False):
        """always_agent=True: the one-launch top-k kernel reads every row's hand-over with
        agent-scope loads, as it does for a row whose workgroups ran on different XCDs."""
        self._check(self.lib.geist_hip_sampler_handoff_scope(self.h, 1 if always_agent else 0))

    def notify_ids(self, enable=True):
        """Every sampling call reports into page-locked memory when its ids are written."""
        self._check(self.lib.geist_hip_sampler_notify_ids(self.h, 1 if enable else 0))

    def wait_ids(self):
        """Returns when the ids of the last sampling call are written (see notify_ids)."""
        self._check(self.lib.geist_hip_sampler_wait_ids(self.h))

    def set_sums(self, fast=False):
        """The sums of exponentials bit-exact (default) or from the hardware's 2^z
        (geist_hip_sampler_set_sums)."""
        self._check(self.lib.geist_hip_sampler_set_sums(self.h, 1 if fast else 0))

    def set_wait_spin(self, microseconds):
        self._check(self.lib.geist_hip_sampler_set_wait_spin(self.h, microseconds))

    def one_launch_spec(self, enable=True):
        """Whether stochastic verification sums the residual and draws in one launch for
        batches that qualify."""
        rc = self.lib.geist_hip_sampler_one_launch_spec(self.h, 1 if enable else 0)
        if rc < 0:
            self._check(rc)
        return bool(rc)

    def prepare(self, params, n_vocab=0):
        """Sizes whatever workspace `params` needs beyond the sampler's own, ahead of the first
        sampling call (the reference does so when a session's options are applied)."""
        self._check(self.lib.geist_hip_sampler_prepare(self.h, C.byref(params), int(n_vocab)))

    def set_stream(self, stream_ptr):
        self._check(self.lib.geist_hip_sampler_set_stream(self.h, stream_ptr))

    def sync(self):
        self._check(self.lib.geist_hip_sampler_sync(self.h))

    def host_buffer(self, nbytes):
        return HostBuffer(self, nbytes)

    def set_logits_hint(self, streamed):
        """streamed=True: the rows come from HBM and are read once (non-temporal loads in the
        single-pass modes); False (default): they may still be cache-resident."""
        self._check(self.lib.geist_hip_sampler_set_logits_hint(self.h, int(streamed)))

    @staticmethod
    def rows(logits, history=None, history_len=None, n_vocab=None, allowed=None):
        """logits: 2-D float32 device tensor (row stride = logits.stride(0)). allowed: 2-D int32
        device tensor of mask words, one row per logit row or a single row shared by all."""
        assert logits.dim() == 2 and logits.stride(1) == 1
        r = Rows()
        r.d_logits = logits.data_ptr()
        r.ld = logits.stride(0) if logits.shape[0] > 1 else max(logits.stride(0), logits.shape[1])
        r.rows = logits.shape[0]
        r.n_vocab = n_vocab if n_vocab is not None else logits.shape[1]
        if history is not None:
            assert history.dim() == 2 and history.stride(1) == 1
            r.d_history = history.data_ptr()
            r.history_ld = history.stride(0) if history.shape[0] > 1 else history.shape[1]
            r.d_history_len = history_len.data_ptr()
        if allowed is not None:
            assert allowed.dim() == 2 and allowed.stride(1) == 1 and allowed.element_size() == 4
            assert allowed.shape[0] in (1, r.rows) and allowed.shape[1] * 32 >= r.n_vocab
            r.d_allowed = allowed.data_ptr()
            r.allowed_ld = 0 if allowed.shape[0] == 1 else allowed.stride(0)
        return r

    def sample(self, rows, params, uniforms, out):
        self._check(self.lib.geist_hip_sample_rows(self.h, C.byref(rows), C.byref(params),
                                                   _ptr(uniforms), _ptr(out)))

    def sample_rng(self, rows, params, states, shared, out):
        self._check(self.lib.geist_hip_sample_rows_rng(self.h, C.byref(rows), C.byref(params),
                                                       _ptr(states), int(shared), _ptr(out)))

    def argmax_f32(self, logits_row):
        idx = C.c_int32(-1)
        self._check(self.lib.geist_hip_argmax_f32(self.h, _ptr(logits_row), logits_row.numel(),
                                                  C.byref(idx)))
        return idx.value

    def apply_penalties(self, logits, history, history_len, rep, freq, pres):
        ld = logits.stride(0) if logits.shape[0] > 1 else logits.shape[1]
        hld = history.stride(0) if history.shape[0] > 1 else history.shape[1]
        self._check(self.lib.geist_hip_apply_penalties(self.h, _ptr(logits), ld, logits.shape[0],
                                                       logits.shape[1], _ptr(history), hld,
                                                       _ptr(history_len), rep, freq, pres))

    def softmax(self, rows, params, probs):
        ld = probs.stride(0) if probs.shape[0] > 1 else probs.shape[1]
        self._check(self.lib.geist_hip_softmax_rows(self.h, C.byref(rows), C.byref(params),
                                                    _ptr(probs), ld))

    def spec_verify(self, target, q, draft, uniforms, temperature, out_tokens, n_accepted,
                    softcap=0.0):
        """q = None: point-mass drafts (the drafter proposed each token with certainty)."""
        n_seq, lp1, n = target.shape
        L = lp1 - 1
        assert draft.shape == (n_seq, L) and target.is_contiguous()
        assert q is None or (q.shape == (n_seq, L, n) and q.is_contiguous())
        self._check(self.lib.geist_hip_spec_verify(self.h, _ptr(target), n, _ptr(q), n, _ptr(draft),
                                                   _ptr(uniforms), n_seq, L, n, temperature,
                                                   softcap, _ptr(out_tokens), _ptr(n_accepted)))

    def propose_drafts_ngram(self, history, history_len, seeds, k_max, max_suffix, out_drafts,
                             out_count, out_match_len):
        """N-gram drafts for every sequence: history [n_seq, H] int32 with history_len [n_seq],
        seeds [n_seq]; out_drafts [n_seq, >= k_max], out_count and out_match_len [n_seq]."""
        n_seq = history.shape[0]
        hld = history.stride(0) if n_seq > 1 else history.shape[1]
        old = out_drafts.stride(0) if n_seq > 1 else out_drafts.shape[1]
        self._check(self.lib.geist_hip_propose_drafts_ngram(
            self.h, _ptr(history), hld, _ptr(history_len), _ptr(seeds), n_seq, int(k_max),
            int(max_suffix), _ptr(out_drafts), old, _ptr(out_count), _ptr(out_match_len)))

    def rmsnorm(self, x, weight, eps, y):
        """x, y: [rows, n] float32 device tensors (y may be x); weight: [n]."""
        rows, n = x.shape
        self._check(self.lib.geist_hip_rmsnorm_rows(self.h, _ptr(x), x.stride(0) if rows > 1 else n,
                                                    _ptr(weight), eps, rows, n, _ptr(y),
                                                    y.stride(0) if rows > 1 else n))

    def f16_gemv(self, w_f16, x, y):
        """w_f16: [n_out, n_in] float16 (or int16 bit patterns), x: [m, n_in] float32,
        y: [m, n_out] float32: y[m] = W x[m] in the reference's order of summation."""
        n_out, n_in = w_f16.shape
        m = x.shape[0]
        assert w_f16.is_contiguous() and w_f16.element_size() == 2 and x.shape[1] == n_in
        self._check(self.lib.geist_hip_f16_gemv_rows(
            self.h, _ptr(w_f16), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def set_projection(self, portable):
        """Which reference backend project_sample's projection stands for: False / 0 the x86
        backend (on a host with AVX-512), True / 1 the portable one, 2 x86 without AVX-512."""
        self._check(self.lib.geist_hip_sampler_set_projection(self.h, int(portable)))

    def f16_linear(self, w_f16, x, y):
        """As f16_gemv in the portable kernel's arithmetic: the sum in double, rounded once."""
        n_out, n_in = w_f16.shape
        m = x.shape[0]
        assert w_f16.is_contiguous() and w_f16.element_size() == 2 and x.shape[1] == n_in
        self._check(self.lib.geist_hip_f16_linear_rows(
            self.h, _ptr(w_f16), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q6k_linear(self, w_q6k, n_in, x, y):
        """w_q6k: uint8 [n_out, n_in / 256 * 210], the Q6_K super-blocks of each table row; the
        portable kernel's arithmetic (sum in double in index order, rounded once)."""
        n_out = w_q6k.shape[0]
        m = x.shape[0]
        assert w_q6k.is_contiguous() and w_q6k.element_size() == 1 and x.shape[1] == n_in
        assert w_q6k.shape[1] == n_in // 256 * 210
        self._check(self.lib.geist_hip_q6k_linear_rows(
            self.h, _ptr(w_q6k), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q6k_packed_bytes(self, n_out, n_in):
        return int(self.lib.geist_hip_q6k_packed_bytes(n_out, n_in))

    def q6k_pack(self, w_q6k, n_in, packed):
        """packed: uint8 tensor of q6k_packed_bytes(n_out, n_in) bytes, 16-byte aligned."""
        n_out = w_q6k.shape[0]
        assert packed.numel() * packed.element_size() >= self.q6k_packed_bytes(n_out, n_in)
        self._check(self.lib.geist_hip_q6k_pack(self.h, _ptr(w_q6k), n_out, n_in, _ptr(packed)))

    def q6k_packed_linear(self, packed, n_out, n_in, x, y):
        m = x.shape[0]
        self._check(self.lib.geist_hip_q6k_packed_linear_rows(
            self.h, _ptr(packed), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q6k_packed_gemv_x86(self, packed, n_out, n_in, x, y):
        """The x86 backend's integer decode kernel over the packed copy, row by row."""
        m = x.shape[0]
        self._check(self.lib.geist_hip_q6k_packed_gemv_x86_rows(
            self.h, _ptr(packed), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q6k_gemv_x86(self, w_q6k, n_in, x, y):
        """The x86 backend's integer decode kernel over the table as it lies in the file."""
        n_out, m = w_q6k.shape[0], x.shape[0]
        assert w_q6k.is_contiguous() and w_q6k.shape[1] == n_in // 256 * 210
        self._check(self.lib.geist_hip_q6k_gemv_x86_rows(
            self.h, _ptr(w_q6k), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q4k_packed_gemv_x86(self, packed, n_out, n_in, x, y):
        """The x86 backend's integer decode kernel over the packed Q4_K copy, row by row."""
        m = x.shape[0]
        self._check(self.lib.geist_hip_q4k_packed_gemv_x86_rows(
            self.h, _ptr(packed), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q6k_packed_linear_x86(self, packed, n_out, n_in, x, y):
        """The x86 backend's projection of a batch over the packed Q6_K copy
        (cpu_x86_linear_q6k_mN; one row: the decode kernel)."""
        m = x.shape[0]
        self._check(self.lib.geist_hip_q6k_packed_linear_x86_rows(
            self.h, _ptr(packed), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q6k_linear_x86(self, w_q6k, n_in, x, y):
        """The same over the table as it lies in the file."""
        n_out, m = w_q6k.shape[0], x.shape[0]
        assert w_q6k.is_contiguous() and w_q6k.shape[1] == n_in // 256 * 210
        self._check(self.lib.geist_hip_q6k_linear_x86_rows(
            self.h, _ptr(w_q6k), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q4k_packed_linear_x86(self, packed, n_out, n_in, x, y):
        """The x86 backend's projection of a batch over the packed Q4_K copy
        (cpu_x86_linear_q4k_mN; one row: the decode kernel)."""
        m = x.shape[0]
        self._check(self.lib.geist_hip_q4k_packed_linear_x86_rows(
            self.h, _ptr(packed), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def q8k_act_bytes(self, n_in, n_rows=1):
        return int(self.lib.geist_hip_q8k_act_bytes(n_in, n_rows))

    def q8k_quantize(self, x, act):
        """x [m, n_in] float32 -> act: the rows as int8 super-blocks (q8k_act_bytes bytes)."""
        m, n_in = x.shape
        assert act.numel() * act.element_size() >= self.q8k_act_bytes(n_in, m)
        self._check(self.lib.geist_hip_q8k_quantize_rows(
            self.h, _ptr(x), x.stride(0) if m > 1 else n_in, m, n_in, _ptr(act)))

    def q6k_packed_gemv_q8k(self, packed, n_out, n_in, act, y):
        """One row of int8 activations (q8k_quantize) times the packed table: y [n_out]."""
        self._check(self.lib.geist_hip_q6k_packed_gemv_q8k(self.h, _ptr(packed), n_out, n_in,
                                                           _ptr(act), _ptr(y)))

    def q8k_row_act_bytes(self, n_in):
        return int(self.lib.geist_hip_q8k_row_act_bytes(n_in))

    def q8k_row_quantize(self, x, act):
        """x [n_in] float32 -> act: the row as int8 with one scale (q8k_row_act_bytes bytes)."""
        n_in = x.numel()
        assert x.is_contiguous() and act.numel() * act.element_size() >= self.q8k_row_act_bytes(n_in)
        self._check(self.lib.geist_hip_q8k_row_quantize(self.h, _ptr(x), n_in, _ptr(act)))

    def q4k_packed_gemv_q8k(self, packed, n_out, n_in, act, y):
        """One row of int8 activations (q8k_row_quantize) times the packed Q4_K table: y [n_out]."""
        self._check(self.lib.geist_hip_q4k_packed_gemv_q8k(self.h, _ptr(packed), n_out, n_in,
                                                           _ptr(act), _ptr(y)))

    def f16_to_q8w(self, w_f16, wq, scales):
        """w_f16 [n_out, n_in] float16 -> wq int8 [n_out, n_in], scales float32 [n_out]."""
        n_out, n_in = w_f16.shape
        self._check(self.lib.geist_hip_f16_to_q8w(self.h, _ptr(w_f16), n_out, n_in, _ptr(wq),
                                                  _ptr(scales)))

    def q8w_gemv(self, wq, scales, x, y):
        n_out, n_in = wq.shape
        m = x.shape[0]
        assert wq.is_contiguous() and wq.element_size() == 1
        self._check(self.lib.geist_hip_q8w_gemv_rows(
            self.h, _ptr(wq), _ptr(scales), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in,
            m, _ptr(y), y.stride(0) if m > 1 else n_out))

    def project_sample(self, hidden, norm_w, eps, embed_f16, logits, params, uniforms, out,
                       normed=None, rng_states=None, shared=True):
        """Norm -> F16 lm_head -> sampler for hidden [rows, d_model]; logits [rows, vocab] is
        written on the way."""
        rows, d_model = hidden.shape
        vocab = embed_f16.shape[0]
        self._check(self.lib.geist_hip_project_sample_rows(
            self.h, _ptr(hidden), hidden.stride(0) if rows > 1 else d_model, rows, d_model,
            _ptr(norm_w), eps, _ptr(embed_f16), vocab, _ptr(normed), _ptr(logits),
            logits.stride(0) if rows > 1 else vocab, C.byref(params), _ptr(uniforms),
            _ptr(rng_states), int(shared), _ptr(out)))

    def project_sample_q8w(self, hidden, norm_w, eps, embed_q8, scales, logits, params, uniforms,
                           out, normed=None, rng_states=None, shared=True):
        """project_sample over the int8 table [vocab, d_model] and its per-row scales."""
        rows, d_model = hidden.shape
        vocab = embed_q8.shape[0]
        self._check(self.lib.geist_hip_project_sample_rows_q8w(
            self.h, _ptr(hidden), hidden.stride(0) if rows > 1 else d_model, rows, d_model,
            _ptr(norm_w), eps, _ptr(embed_q8), _ptr(scales), vocab, _ptr(normed), _ptr(logits),
            logits.stride(0) if rows > 1 else vocab, C.byref(params), _ptr(uniforms),
            _ptr(rng_states), int(shared), _ptr(out)))

    def project_sample_q6k(self, hidden, norm_w, eps, embed_q6k, logits, params, uniforms, out,
                           normed=None, rng_states=None, shared=True):
        """project_sample over a Q6_K table: uint8 [vocab, d_model / 256 * 210]."""
        rows, d_model = hidden.shape
        vocab = embed_q6k.shape[0]
        assert embed_q6k.is_contiguous() and embed_q6k.shape[1] == d_model // 256 * 210
        self._check(self.lib.geist_hip_project_sample_rows_q6k(
            self.h, _ptr(hidden), hidden.stride(0) if rows > 1 else d_model, rows, d_model,
            _ptr(norm_w), eps, _ptr(embed_q6k), vocab, _ptr(normed), _ptr(logits),
            logits.stride(0) if rows > 1 else vocab, C.byref(params), _ptr(uniforms),
            _ptr(rng_states), int(shared), _ptr(out)))

    def project_sample_q6k_packed(self, hidden, norm_w, eps, packed, vocab, logits, params,
                                  uniforms, out, normed=None, rng_states=None, shared=True):
        """project_sample over the packed copy of a Q6_K table (q6k_pack)."""
        rows, d_model = hidden.shape
        self._check(self.lib.geist_hip_project_sample_rows_q6k_packed(
            self.h, _ptr(hidden), hidden.stride(0) if rows > 1 else d_model, rows, d_model,
            _ptr(norm_w), eps, _ptr(packed), vocab, _ptr(normed), _ptr(logits),
            logits.stride(0) if rows > 1 else vocab, C.byref(params), _ptr(uniforms),
            _ptr(rng_states), int(shared), _ptr(out)))

    def q4k_packed_bytes(self, n_out, n_in):
        return int(self.lib.geist_hip_q4k_packed_bytes(n_out, n_in))

    def q4k_pack(self, w_q4k, n_in, packed):
        """w_q4k: uint8 [n_out, n_in / 256 * 144]; packed: uint8 tensor of q4k_packed_bytes(n_out,
        n_in) bytes, 16-byte aligned."""
        n_out = w_q4k.shape[0]
        assert packed.numel() * packed.element_size() >= self.q4k_packed_bytes(n_out, n_in)
        self._check(self.lib.geist_hip_q4k_pack(self.h, _ptr(w_q4k), n_out, n_in, _ptr(packed)))

    def q4k_packed_linear(self, packed, n_out, n_in, x, y):
        m = x.shape[0]
        self._check(self.lib.geist_hip_q4k_packed_linear_rows(
            self.h, _ptr(packed), n_out, n_in, _ptr(x), x.stride(0) if m > 1 else n_in, m, _ptr(y),
            y.stride(0) if m > 1 else n_out))

    def project_sample_q4k_packed(self, hidden, norm_w, eps, packed, vocab, logits, params,
                                  uniforms, out, normed=None, rng_states=None, shared=True):
        """project_sample over the packed copy of a Q4_K table (q4k_pack)."""
        rows, d_model = hidden.shape
        self._check(self.lib.geist_hip_project_sample_rows_q4k_packed(
            self.h, _ptr(hidden), hidden.stride(0) if rows > 1 else d_model, rows, d_model,
            _ptr(norm_w), eps, _ptr(packed), vocab, _ptr(normed), _ptr(logits),
            logits.stride(0) if rows > 1 else vocab, C.byref(params), _ptr(uniforms),
            _ptr(rng_states), int(shared), _ptr(out)))

    def spec_head_geometry(self, vocab, d_model, stride=0, topk=0):
        """(sketch_dim, topk), or None where no sketch head is built."""
        sd, k = C.c_size_t(), C.c_size_t()
        rc = self.lib.geist_hip_spec_head_geometry(vocab, d_model, stride, topk, C.byref(sd),
                                                   C.byref(k))
        return None if rc else (sd.value, k.value)

    def spec_head_build(self, embed_f16, stride=0, topk=0):
        """Handle of the sketch head over the [vocab, d_model] binary16 table."""
        vocab, d_model = embed_f16.shape
        h = C.c_void_p()
        self._check(self.lib.geist_hip_spec_head_build(self.h, _ptr(embed_f16), vocab, d_model,
                                                       stride, topk, C.byref(h)))
        return h

    def spec_head_destroy(self, sh):
        self.lib.geist_hip_spec_head_destroy(self.h, sh)

    def spec_head_view(self, sh):
        v = SpecHeadView()
        self._check(self.lib.geist_hip_spec_head_view(sh, C.byref(v)))
        return v

    def spec_head_try(self, sh, hidden_normed, result, verify=False):
        """result: a device buffer of 24 bytes that receives struct geist_hip_spec_result."""
        self._check(self.lib.geist_hip_spec_head_try(self.h, sh, _ptr(hidden_normed), int(verify),
                                                     _ptr(result)))

    def spec_head_try_hidden(self, sh, hidden, norm_w, eps, normed, result, verify=False):
        """spec_head_try with the output norm in front; normed receives the normed row."""
        self._check(self.lib.geist_hip_spec_head_try_hidden(
            self.h, sh, _ptr(hidden), _ptr(norm_w), eps, _ptr(normed), int(verify), _ptr(result)))

    def logprob(self, logits, tokens, out, softcap=0.0):
        """out[r, j] = log_softmax(logits[r])[tokens[r, j]] (float64), logits soft-capped first
        when softcap > 0."""
        rows, n = logits.shape
        assert tokens.shape == out.shape and tokens.shape[0] == rows
        self._check(self.lib.geist_hip_logprob_rows(
            self.h, _ptr(logits), logits.stride(0), rows, n, softcap, _ptr(tokens),
            tokens.stride(0), tokens.shape[1], _ptr(out), out.stride(0)))

    def topk_paths(self, rows):
        """Which path served each row of the last top-k call (0 candidates handed on by the scan,
        1 per-thread maxima, 2 whole row; -1: the call did not take the candidate path)."""
        import numpy as np
        out = np.zeros(int(rows), dtype=np.int32)
        self._check(self.lib.geist_hip_sampler_topk_paths(self.h, out.ctypes.data_as(C.c_void_p),
                                                          int(rows)))
        return out

    def row_paths(self, rows):
        """Which walk served each row of the last full-vocabulary top-p / min-p call
        (1 shortcut, 2 candidate list, 3 whole row)."""
        import numpy as np
        out = np.zeros(int(rows), dtype=np.int32)
        self._check(self.lib.geist_hip_sampler_row_paths(self.h, out.ctypes.data_as(C.c_void_p),
                                                         int(rows)))
        return out
