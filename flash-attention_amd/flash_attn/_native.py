"""ctypes binding of libfa_mi355x.so, shaped like the reference's pybind11 module.

The three functions `fwd`, `varlen_fwd`, `fwd_kvcache` take the same positional arguments and
return the same tensor lists as `flash_attn_2_cuda.fwd / varlen_fwd / fwd_kvcache`
(csrc/flash_attn/flash_api.cpp:248-259, 426-442, 1038-1055, return lists at :423, :584, :1278),
so `flash_attn_interface.py` calls them exactly as the reference does.  What the reference does in
C++ with ATen before its kernels run -- argument checks with the same messages, head-dim padding
to a multiple of 8, output / log-sum-exp / split-accumulator allocation on q's device with the
torch caching allocator, current-stream launch -- happens here; the shared library itself takes
plain pointers and sizes and allocates nothing.

There is no fallback: if the library is missing or cannot be loaded, importing this module fails.
"""
import ctypes
import math
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# FLASH_ATTN_MI355X_LIB selects another build of the same library (kernel tuning experiments).
_LIB_PATH = os.environ.get("FLASH_ATTN_MI355X_LIB") or os.path.join(_HERE, "libfa_mi355x.so")

FA_DTYPE_FP16 = 0
FA_DTYPE_BF16 = 1
FA_DTYPE_FP32 = 2


class FaFwdParams(ctypes.Structure):
    """Mirror of `fa_fwd_params` in include/fa_mi355x.h (field order matters)."""
    _fields_ = (
        [(n, ctypes.c_void_p) for n in (
            "q", "k", "v", "o", "softmax_lse", "o_accum", "lse_accum", "k_new", "v_new",
            "rotary_cos", "rotary_sin", "cu_seqlens_q", "cu_seqlens_k", "cache_batch_idx", "work_counter")]
        + [(n, ctypes.c_int64) for n in (
            "q_batch_stride", "q_row_stride", "q_head_stride",
            "k_batch_stride", "k_row_stride", "k_head_stride",
            "v_batch_stride", "v_row_stride", "v_head_stride",
            "o_batch_stride", "o_row_stride", "o_head_stride",
            "knew_batch_stride", "knew_row_stride", "knew_head_stride",
            "vnew_batch_stride", "vnew_row_stride", "vnew_head_stride")]
        + [(n, ctypes.c_int32) for n in (
            "b", "h", "h_k", "seqlen_q", "seqlen_k", "seqlen_knew", "d", "rotary_dim",
            "window_left", "window_right", "is_causal", "is_seqlens_k_cumulative",
            "is_rotary_interleaved", "num_splits", "dtype")]
        + [("softmax_scale", ctypes.c_float), ("p_dropout", ctypes.c_float),
           ("rng_state", ctypes.c_void_p), ("s_dmask", ctypes.c_void_p),
           ("sdm_rows", ctypes.c_int32), ("sdm_cols", ctypes.c_int32),
           ("work_counter_len", ctypes.c_int32), ("reserved0", ctypes.c_int32)]
    )


class FaRotaryParams(ctypes.Structure):
    """Mirror of `fa_rotary_params` in include/fa_mi355x.h (field order matters)."""
    _fields_ = (
        [(n, ctypes.c_void_p) for n in ("x", "out", "cos", "sin", "cu_seqlens", "seqlen_offsets")]
        + [(n, ctypes.c_int64) for n in (
            "x_batch_stride", "x_row_stride", "x_head_stride",
            "o_batch_stride", "o_row_stride", "o_head_stride", "cs_row_stride")]
        + [(n, ctypes.c_int32) for n in (
            "b", "seqlen", "h", "d", "rotary_dim", "seqlen_ro", "seqlen_offset",
            "interleaved", "conjugate", "dtype", "cs_dtype")]
    )


class FaBwdParams(ctypes.Structure):
    """Mirror of `fa_bwd_params` in include/fa_mi355x.h (field order matters)."""
    _fields_ = (
        [(n, ctypes.c_void_p) for n in ("dout", "q", "k", "v", "out", "softmax_lse", "dq", "dk", "dv",
                                        "softmax_d", "cu_seqlens_q", "cu_seqlens_k")]
        + [("%s_%s_stride" % (t, a), ctypes.c_int64) for t in ("q", "k", "v", "o", "do", "dq", "dk", "dv")
           for a in ("batch", "row", "head")]
        + [(n, ctypes.c_int32) for n in ("b", "seqlen_q", "seqlen_k", "h", "h_k", "d", "seqlen_q_rounded")]
        + [("softmax_scale", ctypes.c_float)]
        + [(n, ctypes.c_int32) for n in ("is_causal", "window_left", "window_right", "dtype")]
        + [("p_dropout", ctypes.c_float), ("rng_state", ctypes.c_void_p)]
    )


def _load():
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            "flash_attn: %s not found. Build it with `python flash-attention_amd/build.py` "
            "(hipcc, gfx950). There is no fallback implementation." % _LIB_PATH)
    lib = ctypes.CDLL(_LIB_PATH)
    P = ctypes.POINTER(FaFwdParams)
    for name in ("fa_fwd", "fa_varlen_fwd", "fa_fwd_kvcache", "fa_fwd_kvcache_noalloc"):
        f = getattr(lib, name)
        f.argtypes = [P, ctypes.c_void_p]
        f.restype = ctypes.c_int
    lib.fa_plan_splits.argtypes = [P, ctypes.c_int32, ctypes.POINTER(ctypes.c_int32)]
    lib.fa_work_list_words.argtypes = [P]
    lib.fa_work_list_words.restype = ctypes.c_int64
    lib.fa_plan_splits.restype = ctypes.c_int
    lib.fa_num_splits_heuristic_reference.argtypes = [ctypes.c_int32] * 4
    lib.fa_num_splits_heuristic_reference.restype = ctypes.c_int
    lib.fa_set_rng_state.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_void_p]
    lib.fa_set_rng_state.restype = ctypes.c_int
    lib.fa_last_error.argtypes = []
    lib.fa_last_error.restype = ctypes.c_char_p
    lib.fa_version.argtypes = []
    lib.fa_version.restype = ctypes.c_int32
    lib.fa_last_kernel.argtypes = []
    lib.fa_last_kernel.restype = ctypes.c_int32
    lib.fa_sizeof_params.argtypes = []
    lib.fa_sizeof_params.restype = ctypes.c_int32
    for name in ("fa_bwd", "fa_varlen_bwd"):
        f = getattr(lib, name)
        f.argtypes = [ctypes.POINTER(FaBwdParams), ctypes.c_void_p]
        f.restype = ctypes.c_int
    lib.fa_sizeof_bwd_params.argtypes = []
    lib.fa_sizeof_bwd_params.restype = ctypes.c_int32
    if lib.fa_sizeof_bwd_params() != ctypes.sizeof(FaBwdParams):
        raise ImportError("flash_attn: fa_bwd_params layout mismatch between %s and its Python mirror; "
                          "rebuild the library" % _LIB_PATH)
    lib.fa_rotary.argtypes = [ctypes.POINTER(FaRotaryParams), ctypes.c_void_p]
    lib.fa_rotary.restype = ctypes.c_int
    lib.fa_sizeof_rotary_params.argtypes = []
    lib.fa_sizeof_rotary_params.restype = ctypes.c_int32
    if lib.fa_sizeof_rotary_params() != ctypes.sizeof(FaRotaryParams):
        raise ImportError("flash_attn: fa_rotary_params layout mismatch between %s and its Python mirror; "
                          "rebuild the library" % _LIB_PATH)
    if lib.fa_sizeof_params() != ctypes.sizeof(FaFwdParams):
        raise ImportError("flash_attn: fa_fwd_params layout mismatch between %s (%d bytes) and its "
                          "Python mirror (%d bytes); rebuild the library" %
                          (_LIB_PATH, lib.fa_sizeof_params(), ctypes.sizeof(FaFwdParams)))
    return lib


lib = _load()


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _call(fn, params, stream, device=None):
    rc = fn(ctypes.byref(params), ctypes.c_void_p(stream))
    if rc != 0:
        msg = lib.fa_last_error().decode() or "libfa_mi355x: error %d" % rc
        if device is not None:
            _reset_counters(device)
        raise RuntimeError(msg)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _dtype_code(dtype):
    _check(dtype in (torch.float16, torch.bfloat16), "FlashAttention only support fp16 and bf16 data type")
    return FA_DTYPE_BF16 if dtype == torch.bfloat16 else FA_DTYPE_FP16


def _check_device(*ts):
    for t in ts:
        _check(t.is_cuda, "Input tensor must be on CUDA device")


def _pad8(t):
    d = t.shape[-1]
    return t if d % 8 == 0 else torch.nn.functional.pad(t, (0, 8 - d % 8))


def _round_up(x, m):
    return (x + m - 1) // m * m


def _stream(device):
    """raw handle of torch's current stream on `device` (what `torch.cuda.current_stream(device).cuda_stream`
    returns, without building the Stream object: this runs twice per call)"""
    index = device.index
    return torch._C._cuda_getCurrentRawStream(index if index is not None else torch.cuda.current_device())


class _on_device:
    """`with torch.cuda.device(device)` that costs nothing when `device` is already the current one (the guard is
    only there for callers that pass tensors of another GPU than the current)."""
    __slots__ = ("guard",)

    def __init__(self, device):
        index = device.index
        self.guard = None if index is None or index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


_NO_DROPOUT_STATE = {}     # device -> the (never read, never written) rng_state returned when p_dropout = 0


def _dropout_state(p, p_dropout, return_softmax, gen_, batch, heads, seqlen_q, seqlen_k, dtype, device):
    """Seed / offset of the dropout mask taken from (and advancing) torch's generator for the device,
    like the reference does with its Philox state (flash_api.cpp:396-408), and the optional
    probability tensor behind return_softmax (:351-357).  Returns (rng_state, s_dmask).

    Without dropout nothing is allocated: one placeholder tensor per device stands in for the
    reference's empty rng_state.  With dropout the two words reach the device as arguments of a
    one-thread kernel on the current stream (no pageable copy, no host synchronisation).  Under HIP
    graph capture the generator cannot be advanced from the host per replay, so dropout is refused
    there."""
    _check(0.0 <= p_dropout < 1.0, "p_dropout must be in [0, 1)")
    s_dmask = None
    if return_softmax:
        _check(p_dropout > 0.0, "return_softmax is only supported when p_dropout > 0.0")
        s_dmask = torch.empty((batch, heads, _round_up(seqlen_q, 128), _round_up(seqlen_k, 128)), dtype=dtype, device=device)
        p.s_dmask, p.sdm_rows, p.sdm_cols = s_dmask.data_ptr(), s_dmask.shape[2], s_dmask.shape[3]
    if p_dropout <= 0.0:
        key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
        if key not in _NO_DROPOUT_STATE:
            _NO_DROPOUT_STATE[key] = torch.empty((2,), dtype=torch.int64, device=device)
        return _NO_DROPOUT_STATE[key], s_dmask
    _check(not torch.cuda.is_current_stream_capturing(),
           "attention dropout cannot be captured in a HIP graph: its seed and offset come from the host-side generator")
    rng_state = torch.empty((2,), dtype=torch.int64, device=device)
    gen = gen_ if gen_ is not None else torch.cuda.default_generators[device.index if device.index is not None
                                                                   else torch.cuda.current_device()]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + batch * heads * 32)
    rc = lib.fa_set_rng_state(ctypes.c_void_p(rng_state.data_ptr()), ctypes.c_uint64(seed & (2 ** 64 - 1)),
                              ctypes.c_uint64(offset & (2 ** 64 - 1)), ctypes.c_void_p(_stream(device)))
    if rc != 0:
        raise RuntimeError(lib.fa_last_error().decode() or "libfa_mi355x: error %d" % rc)
    p.p_dropout, p.rng_state = p_dropout, rng_state.data_ptr()
    return rng_state, s_dmask


WORK_COUNTER_WORDS = 4      # FA_WORK_COUNTER_WORDS of include/fa_mi355x.h
_COUNTERS = {}     # (device index, stream) -> int32 words lent to the ticket-scheduled kernels


_RETIRED = []
WORK_LIST = True      # packed forward launches lend the library room for its device-built work list


def _counters(device, words):
    """Counter words for launches on the current stream of `device`: zero when first handed out and left
    zero by every launch, so one tensor per (device, stream) serves all calls (launches on one stream do
    not overlap).  The kernels tag the words with a number of the call and treat anything else they find as
    zero, so a tensor that has to be made while the stream is capturing a HIP graph is handed out uncleared:
    the graph then holds no fill of it."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (index, _stream(device))
    t = _COUNTERS.get(key)
    if t is None or t.numel() < words:
        if t is not None:
            _RETIRED.append(t)      # a captured graph may still point at it
        make = torch.empty if torch.cuda.is_current_stream_capturing() else torch.zeros
        t = make((max(16, int(words)),), dtype=torch.int32, device=device)
        _COUNTERS[key] = t
    return t


def _reset_counters(device):
    """After a call that returned an error: clear the counter words of the device's streams (a launch that did
    not complete may have left them in use; the next launch would cope, this keeps them tidy)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if torch.cuda.is_current_stream_capturing():
        return
    for (dev, _), t in _COUNTERS.items():
        if dev == index:
            t[:WORK_COUNTER_WORDS].zero_()


def _plan_and_alloc(params, api, batch, heads, seqlen_q, d, device):
    """Resolve the split count and allocate the fp32 partial buffers like the reference does
    (flash_api.cpp:373-389, 1241-1257).  The returned tensors must stay alive until launch."""
    n = ctypes.c_int32(0)
    counter = _counters(device, WORK_COUNTER_WORDS)
    params.work_counter = counter.data_ptr()
    params.work_counter_len = counter.numel()
    rc = lib.fa_plan_splits(ctypes.byref(params), api, ctypes.byref(n))
    if rc != 0:
        raise RuntimeError(lib.fa_last_error().decode())
    keep = (counter,)
    if n.value > 1:
        lse_accum = torch.empty((n.value, batch, heads, seqlen_q), dtype=torch.float32, device=device)
        o_accum = torch.empty((n.value, batch, heads, seqlen_q, _round_up(d, 32)), dtype=torch.float32, device=device)
        params.lse_accum = lse_accum.data_ptr()
        params.o_accum = o_accum.data_ptr()
        keep = (counter, lse_accum, o_accum)
    return keep


def fwd(q, k, v, out_, p_dropout, softmax_scale, is_causal, window_size_left, window_size_right,
        return_softmax, gen_):
    """Dense batch forward; mirrors mha_fwd (flash_api.cpp:248-424)."""
    q_dtype = q.dtype
    dt = _dtype_code(q_dtype)
    _check(k.dtype == q_dtype, "query and key must have the same dtype")
    _check(v.dtype == q_dtype, "query and value must have the same dtype")
    _check_device(q, k, v)
    for t in (q, k, v):
        _check(t.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    _check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be 4-dimensional")
    batch_size, seqlen_q, num_heads, head_size_og = q.shape
    seqlen_k, num_heads_k = k.shape[1], k.shape[2]
    _check(batch_size > 0, "batch size must be postive")
    _check(head_size_og <= 256, "FlashAttention forward only supports head dimension at most 256")
    _check(num_heads % num_heads_k == 0, "Number of heads in key/value must divide number of heads in query")
    _check(tuple(k.shape) == (batch_size, seqlen_k, num_heads_k, head_size_og), "k must have shape (batch_size, seqlen_k, num_heads_k, head_size)")
    _check(tuple(v.shape) == (batch_size, seqlen_k, num_heads_k, head_size_og), "v must have shape (batch_size, seqlen_k, num_heads_k, head_size)")
    if seqlen_q == 1:
        is_causal = False
    if is_causal:
        window_size_right = 0

    q_padded, k_padded, v_padded = _pad8(q), _pad8(k), _pad8(v)
    if out_ is not None:
        out = out_
        _check(out.dtype == q_dtype, "Output must have the same dtype as inputs")
        _check_device(out)
        _check(out.stride(-1) == 1, "Output tensor must have contiguous last dimension")
        _check(tuple(out.shape) == (batch_size, seqlen_q, num_heads, head_size_og), "out has the wrong shape")
        if head_size_og % 8 != 0:
            out = torch.empty_like(q_padded)
    else:
        out = torch.empty_like(q_padded)
    head_size = q_padded.shape[-1]

    with _on_device(q.device):
        softmax_lse = torch.empty((batch_size, num_heads, seqlen_q), dtype=torch.float32, device=q.device)
        p = FaFwdParams()
        p.q, p.k, p.v, p.o = q_padded.data_ptr(), k_padded.data_ptr(), v_padded.data_ptr(), out.data_ptr()
        p.softmax_lse = softmax_lse.data_ptr()
        p.q_batch_stride, p.q_row_stride, p.q_head_stride = q_padded.stride(0), q_padded.stride(1), q_padded.stride(2)
        p.k_batch_stride, p.k_row_stride, p.k_head_stride = k_padded.stride(0), k_padded.stride(1), k_padded.stride(2)
        p.v_batch_stride, p.v_row_stride, p.v_head_stride = v_padded.stride(0), v_padded.stride(1), v_padded.stride(2)
        p.o_batch_stride, p.o_row_stride, p.o_head_stride = out.stride(0), out.stride(1), out.stride(2)
        p.b, p.h, p.h_k = batch_size, num_heads, num_heads_k
        p.seqlen_q, p.seqlen_k, p.d = seqlen_q, seqlen_k, head_size
        p.window_left, p.window_right, p.is_causal = window_size_left, window_size_right, int(is_causal)
        p.is_seqlens_k_cumulative = 1
        p.num_splits = 0
        p.dtype = dt
        p.softmax_scale = softmax_scale
        rng_state, s_dmask = _dropout_state(p, p_dropout, return_softmax, gen_, batch_size, num_heads, seqlen_q,
                                            seqlen_k, q_dtype, q.device)
        if seqlen_q > 0 and seqlen_k > 0:
            keep = _plan_and_alloc(p, 0, batch_size, num_heads, seqlen_q, head_size, q.device)
            _call(lib.fa_fwd, p, _stream(q.device), q.device)
            del keep
        else:
            out.zero_()
            softmax_lse.fill_(float("inf"))
            if s_dmask is not None:
                s_dmask.zero_()

    out_padded = out
    if head_size_og % 8 != 0:
        out = out[..., :head_size_og]
        if out_ is not None:
            out_.copy_(out)
    return [out, q_padded, k_padded, v_padded, out_padded, softmax_lse, s_dmask, rng_state]


def varlen_fwd(q, k, v, out_, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, p_dropout,
               softmax_scale, zero_tensors, is_causal, window_size_left, window_size_right,
               return_softmax, gen_):
    """Packed variable-length forward; mirrors mha_varlen_fwd (flash_api.cpp:426-585)."""
    q_dtype = q.dtype
    dt = _dtype_code(q_dtype)
    _check(k.dtype == q_dtype, "query and key must have the same dtype")
    _check(v.dtype == q_dtype, "query and value must have the same dtype")
    _check(cu_seqlens_q.dtype == torch.int32, "cu_seqlens_q must have dtype int32")
    _check(cu_seqlens_k.dtype == torch.int32, "cu_seqlens_k must have dtype int32")
    _check_device(q, k, v, cu_seqlens_q, cu_seqlens_k)
    for t in (q, k, v):
        _check(t.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    _check(cu_seqlens_q.is_contiguous(), "cu_seqlens_q must be contiguous")
    _check(cu_seqlens_k.is_contiguous(), "cu_seqlens_k must be contiguous")
    _check(q.dim() == 3 and k.dim() == 3 and v.dim() == 3, "q, k, v must be 3-dimensional")
    total_q, num_heads, head_size_og = q.shape
    total_k, num_heads_k = k.shape[0], k.shape[1]
    batch_size = cu_seqlens_q.numel() - 1
    _check(batch_size > 0, "batch size must be positive")
    _check(head_size_og <= 256, "FlashAttention forward only supports head dimension at most 256")
    _check(num_heads % num_heads_k == 0, "Number of heads in key/value must divide number of heads in query")
    _check(tuple(k.shape) == (total_k, num_heads_k, head_size_og), "k must have shape (total_k, num_heads_k, head_size)")
    _check(tuple(v.shape) == (total_k, num_heads_k, head_size_og), "v must have shape (total_k, num_heads_k, head_size)")
    _check(tuple(cu_seqlens_q.shape) == (batch_size + 1,), "cu_seqlens_q must have shape (batch_size + 1)")
    _check(tuple(cu_seqlens_k.shape) == (batch_size + 1,), "cu_seqlens_k must have shape (batch_size + 1)")
    if is_causal:
        window_size_right = 0

    q_padded, k_padded, v_padded = _pad8(q), _pad8(k), _pad8(v)
    if out_ is not None:
        out = out_
        _check(out.dtype == q_dtype, "Output must have the same dtype as inputs")
        _check_device(out)
        _check(out.stride(-1) == 1, "Output tensor must have contiguous last dimension")
        _check(tuple(out.shape) == (total_q, num_heads, head_size_og), "out has the wrong shape")
        if head_size_og % 8 != 0:
            out = torch.empty_like(q_padded)
    else:
        out = torch.empty_like(q_padded)
    head_size = q_padded.shape[-1]

    with _on_device(q.device):
        softmax_lse = torch.empty((batch_size, num_heads, max_seqlen_q), dtype=torch.float32, device=q.device)
        if zero_tensors:
            out.zero_()
            softmax_lse.fill_(float("-inf"))
        p = FaFwdParams()
        p.q, p.k, p.v, p.o = q_padded.data_ptr(), k_padded.data_ptr(), v_padded.data_ptr(), out.data_ptr()
        p.softmax_lse = softmax_lse.data_ptr()
        p.cu_seqlens_q, p.cu_seqlens_k = cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr()
        p.q_row_stride, p.q_head_stride = q_padded.stride(0), q_padded.stride(1)
        p.k_row_stride, p.k_head_stride = k_padded.stride(0), k_padded.stride(1)
        p.v_row_stride, p.v_head_stride = v_padded.stride(0), v_padded.stride(1)
        p.o_row_stride, p.o_head_stride = out.stride(0), out.stride(1)
        p.b, p.h, p.h_k = batch_size, num_heads, num_heads_k
        p.seqlen_q, p.seqlen_k, p.d = max_seqlen_q, max_seqlen_k, head_size
        p.window_left, p.window_right, p.is_causal = window_size_left, window_size_right, int(is_causal)
        p.is_seqlens_k_cumulative = 1
        p.num_splits = 1
        p.dtype = dt
        p.softmax_scale = softmax_scale
        rng_state, s_dmask = _dropout_state(p, p_dropout, return_softmax, gen_, batch_size, num_heads, max_seqlen_q,
                                            max_seqlen_k, q_dtype, q.device)
        if total_q > 0 and max_seqlen_q > 0:
            # room for the work list the library builds from cu_seqlens_q on the device (WORK_LIST = False: the
            # arithmetic order, for tests that compare the two)
            words = lib.fa_work_list_words(ctypes.byref(p)) if WORK_LIST else WORK_COUNTER_WORDS
            counter = _counters(q.device, words)
            p.work_counter, p.work_counter_len = counter.data_ptr(), counter.numel()
            _call(lib.fa_varlen_fwd, p, _stream(q.device), q.device)
        elif s_dmask is not None:
            s_dmask.zero_()

    out_padded = out
    if head_size_og % 8 != 0:
        out = out[..., :head_size_og]
        if out_ is not None:
            out_.copy_(out)
    return [out, q_padded, k_padded, v_padded, out_padded, softmax_lse, s_dmask, rng_state]


def _set_strides(p, name, t):
    """(batch, row, head) element strides of a (b, s, h, d) tensor, or (0, row, head) of a packed (total, h, d) one."""
    st = t.stride()
    b, r, h = (st[0], st[1], st[2]) if t.dim() == 4 else (0, st[0], st[1])
    setattr(p, name + "_batch_stride", b)
    setattr(p, name + "_row_stride", r)
    setattr(p, name + "_head_stride", h)


def _bwd_common(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, p_dropout, what):
    _check(0.0 <= p_dropout < 1.0, "p_dropout must be in [0, 1)")
    q_dtype = q.dtype
    dt = _dtype_code(q_dtype)
    _check(k.dtype == q_dtype, "query and key must have the same dtype")
    _check(v.dtype == q_dtype, "query and value must have the same dtype")
    _check(out.dtype == q_dtype, "query and out must have the same dtype")
    _check(dout.dtype == q_dtype, "query and dout must have the same dtype")
    _check_device(q, k, v, out, dout, softmax_lse)
    for t in (q, k, v):
        _check(t.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    _check(out.stride(-1) == 1, "out tensor must have contiguous last dimension")
    _check(dout.stride(-1) == 1, "dout tensor must have contiguous last dimension")
    head_size_og, head_size = dout.shape[-1], q.shape[-1]
    _check(head_size % 8 == 0, "head_size should be a multiple of 8")
    _check(head_size <= 256, "FlashAttention backward only supports head dimension at most 256")
    _check(q.shape[-2] % k.shape[-2] == 0, "Number of heads in key/value must divide number of heads in query")
    _check(head_size == _round_up(head_size_og, 8), "head_size must be head_size_og rounded to a multiple of 8")
    _check(tuple(k.shape[:-2]) == tuple(v.shape[:-2]) and k.shape[-2:] == v.shape[-2:] and k.shape[-1] == head_size,
           "k and v must have the same shape and q's head size")
    _check(tuple(out.shape) == tuple(q.shape), "out must have the shape of q")
    _check(tuple(dout.shape) == tuple(q.shape[:-1]) + (head_size_og,), "dout must have the shape of out")
    grads = []
    for g_, like, name in ((dq_, q, "dq"), (dk_, k, "dk"), (dv_, v, "dv")):
        if g_ is None:
            g_ = torch.empty_like(like)
        else:
            _check(g_.dtype == q_dtype, name + " must have the same dtype as q")
            _check_device(g_)
            _check(g_.stride(-1) == 1, name + " must have contiguous last dimension")
            _check(tuple(g_.shape) == tuple(like.shape), name + " has the wrong shape")
        grads.append(g_)
    dout_padded = _pad8(dout)
    return dt, dout_padded, grads


def _slice_grads(dq, dk, dv, head_size_og):
    """Gradients at the caller's head size when it was padded to a multiple of 8 (flash_api.cpp:803-807)."""
    if head_size_og % 8 != 0:
        return [dq[..., :head_size_og], dk[..., :head_size_og], dv[..., :head_size_og]]
    return [dq, dk, dv]


def _fill_bwd(p, dout, q, k, v, out, softmax_lse, dq, dk, dv, softmax_d, softmax_scale, is_causal, wl, wr, dt,
              p_dropout=0.0, rng_state=None):
    if p_dropout > 0.0:
        _check(rng_state is not None and rng_state.is_cuda and rng_state.dtype == torch.int64 and rng_state.numel() == 2,
               "rng_state (the forward's, 2 x int64 on the GPU) is required when dropout_p > 0")
        p.p_dropout, p.rng_state = p_dropout, rng_state.data_ptr()
    p.dout, p.q, p.k, p.v, p.out = dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.softmax_lse, p.softmax_d = softmax_lse.data_ptr(), softmax_d.data_ptr()
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    for name, t in (("q", q), ("k", k), ("v", v), ("o", out), ("do", dout), ("dq", dq), ("dk", dk), ("dv", dv)):
        _set_strides(p, name, t)
    p.h, p.h_k, p.d = q.shape[-2], k.shape[-2], q.shape[-1]
    p.softmax_scale = softmax_scale
    p.is_causal, p.window_left, p.window_right = int(is_causal), wl, (0 if is_causal else wr)
    p.dtype = dt


def bwd(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, p_dropout, softmax_scale, is_causal,
        window_size_left, window_size_right, gen_, rng_state):
    """Dense batch backward; mirrors mha_bwd (flash_api.cpp:609-832).  Returns [dq, dk, dv, softmax_d]."""
    _check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must be 4-dimensional")
    dt, dout_padded, (dq, dk, dv) = _bwd_common(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, p_dropout, "bwd")
    batch_size, seqlen_q, num_heads, _ = q.shape
    seqlen_k = k.shape[1]
    _check(batch_size > 0, "batch size must be positive")
    _check(k.shape[0] == batch_size, "k must have q's batch size")
    _check(tuple(softmax_lse.shape) == (batch_size, num_heads, seqlen_q) and softmax_lse.dtype == torch.float32
           and softmax_lse.is_contiguous(), "softmax_lse must be a contiguous fp32 (batch, nheads, seqlen_q) tensor")
    seqlen_q_rounded = _round_up(seqlen_q, 128)
    with _on_device(q.device):
        softmax_d = torch.empty((batch_size, num_heads, seqlen_q_rounded), dtype=torch.float32, device=q.device)
        p = FaBwdParams()
        _fill_bwd(p, dout_padded, q, k, v, out, softmax_lse, dq, dk, dv, softmax_d, softmax_scale, is_causal,
                  window_size_left, window_size_right, dt, p_dropout, rng_state)
        p.b, p.seqlen_q, p.seqlen_k, p.seqlen_q_rounded = batch_size, seqlen_q, seqlen_k, seqlen_q_rounded
        if seqlen_q > 0 and seqlen_k > 0:
            _call(lib.fa_bwd, p, _stream(q.device))
        else:       # nothing to attend to: all gradients are zero
            dq.zero_(); dk.zero_(); dv.zero_(); softmax_d.zero_()
    return _slice_grads(dq, dk, dv, dout.shape[-1]) + [softmax_d]


def varlen_bwd(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
               max_seqlen_k, p_dropout, softmax_scale, zero_tensors, is_causal, window_size_left,
               window_size_right, gen_, rng_state):
    """Packed variable-length backward; mirrors mha_varlen_bwd (flash_api.cpp:834-1036)."""
    _check(q.dim() == 3 and k.dim() == 3 and v.dim() == 3, "q, k, v must be 3-dimensional")
    dt, dout_padded, (dq, dk, dv) = _bwd_common(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, p_dropout, "varlen_bwd")
    _check(cu_seqlens_q.dtype == torch.int32, "cu_seqlens_q must have dtype int32")
    _check(cu_seqlens_k.dtype == torch.int32, "cu_seqlens_k must have dtype int32")
    _check_device(cu_seqlens_q, cu_seqlens_k)
    _check(cu_seqlens_q.is_contiguous(), "cu_seqlens_q must be contiguous")
    _check(cu_seqlens_k.is_contiguous(), "cu_seqlens_k must be contiguous")
    total_q, num_heads, _ = q.shape
    batch_size = cu_seqlens_q.numel() - 1
    _check(batch_size > 0, "batch size must be positive")
    _check(tuple(cu_seqlens_k.shape) == (batch_size + 1,), "cu_seqlens_k must have shape (batch_size + 1)")
    _check(tuple(softmax_lse.shape) == (batch_size, num_heads, max_seqlen_q) and softmax_lse.dtype == torch.float32
           and softmax_lse.is_contiguous(), "softmax_lse must be a contiguous fp32 (batch, nheads, max_seqlen_q) tensor")
    seqlen_q_rounded = _round_up(max_seqlen_q, 128)
    with _on_device(q.device):
        softmax_d = torch.empty((batch_size, num_heads, seqlen_q_rounded), dtype=torch.float32, device=q.device)
        if zero_tensors:
            dq.zero_(); dk.zero_(); dv.zero_(); softmax_d.zero_()
        p = FaBwdParams()
        _fill_bwd(p, dout_padded, q, k, v, out, softmax_lse, dq, dk, dv, softmax_d, softmax_scale, is_causal,
                  window_size_left, window_size_right, dt, p_dropout, rng_state)
        p.cu_seqlens_q, p.cu_seqlens_k = cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr()
        p.b, p.seqlen_q, p.seqlen_k, p.seqlen_q_rounded = batch_size, max_seqlen_q, max_seqlen_k, seqlen_q_rounded
        if max_seqlen_q > 0 and max_seqlen_k > 0 and total_q > 0 and k.shape[0] > 0:
            _call(lib.fa_varlen_bwd, p, _stream(q.device))
        else:
            dq.zero_(); dk.zero_(); dv.zero_(); softmax_d.zero_()
    return _slice_grads(dq, dk, dv, dout.shape[-1]) + [softmax_d]


def fwd_kvcache(q, kcache, vcache, k_, v_, seqlens_k_, rotary_cos_, rotary_sin_, cache_batch_idx_,
                out_, softmax_scale, is_causal, window_size_left, window_size_right,
                is_rotary_interleaved, num_splits, no_alloc=False, lse_=None):
    """KV-cache forward with optional append + rotary; mirrors mha_fwd_kvcache
    (flash_api.cpp:1038-1279).  Returns [out, softmax_lse].

    no_alloc=True calls fa_fwd_kvcache_noalloc: the split accumulators and the ticket words live in
    the library's own device array, and with out_ and lse_ given nothing is allocated here either."""
    q_dtype = q.dtype
    dt = _dtype_code(q_dtype)
    _check(kcache.dtype == q_dtype, "query and key must have the same dtype")
    _check(vcache.dtype == q_dtype, "query and value must have the same dtype")
    _check_device(q, kcache, vcache)
    for t in (q, kcache, vcache):
        _check(t.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    _check(q.dim() == 4 and kcache.dim() == 4 and vcache.dim() == 4, "q, k_cache, v_cache must be 4-dimensional")
    batch_size, seqlen_q, num_heads, head_size_og = q.shape
    batch_size_c, seqlen_k, num_heads_k = kcache.shape[0], kcache.shape[1], kcache.shape[2]
    _check(batch_size > 0, "batch size must be postive")
    _check(head_size_og <= 256, "FlashAttention forward only supports head dimension at most 256")
    _check(num_heads % num_heads_k == 0, "Number of heads in key/value must divide number of heads in query")
    _check(tuple(kcache.shape) == (batch_size_c, seqlen_k, num_heads_k, head_size_og), "k_cache has the wrong shape")
    _check(tuple(vcache.shape) == (batch_size_c, seqlen_k, num_heads_k, head_size_og), "v_cache has the wrong shape")
    if cache_batch_idx_ is None:
        _check(batch_size_c >= batch_size, "k_cache must hold at least batch_size rows")
    if seqlen_q == 1:
        is_causal = False
    if is_causal:
        window_size_right = 0

    padded = head_size_og % 8 != 0
    q_padded, kcache_padded, vcache_padded = _pad8(q), _pad8(kcache), _pad8(vcache)
    if out_ is not None:
        out = out_
        _check(out.dtype == q_dtype, "Output must have the same dtype as inputs")
        _check_device(out)
        _check(out.stride(-1) == 1, "Output tensor must have contiguous last dimension")
        _check(tuple(out.shape) == (batch_size, seqlen_q, num_heads, head_size_og), "out has the wrong shape")
        if padded:
            out = torch.empty_like(q_padded)
    else:
        out = torch.empty_like(q_padded)
    head_size = q_padded.shape[-1]

    with _on_device(q.device):
        if lse_ is not None:
            _check(lse_.dtype == torch.float32 and lse_.is_contiguous() and tuple(lse_.shape) == (batch_size, num_heads, seqlen_q),
                   "lse_ must be a contiguous fp32 tensor of shape (batch_size, num_heads, seqlen_q)")
            _check_device(lse_)
            softmax_lse = lse_
        else:
            softmax_lse = torch.empty((batch_size, num_heads, seqlen_q), dtype=torch.float32, device=q.device)
        p = FaFwdParams()
        p.q, p.k, p.v, p.o = q_padded.data_ptr(), kcache_padded.data_ptr(), vcache_padded.data_ptr(), out.data_ptr()
        p.softmax_lse = softmax_lse.data_ptr()
        p.q_batch_stride, p.q_row_stride, p.q_head_stride = q_padded.stride(0), q_padded.stride(1), q_padded.stride(2)
        p.k_batch_stride, p.k_row_stride, p.k_head_stride = kcache_padded.stride(0), kcache_padded.stride(1), kcache_padded.stride(2)
        p.v_batch_stride, p.v_row_stride, p.v_head_stride = vcache_padded.stride(0), vcache_padded.stride(1), vcache_padded.stride(2)
        p.o_batch_stride, p.o_row_stride, p.o_head_stride = out.stride(0), out.stride(1), out.stride(2)
        p.b, p.h, p.h_k = batch_size, num_heads, num_heads_k
        p.seqlen_q, p.seqlen_k, p.d = seqlen_q, seqlen_k, head_size
        p.window_left, p.window_right, p.is_causal = window_size_left, window_size_right, int(is_causal)
        p.dtype = dt
        p.softmax_scale = softmax_scale

        keep = []
        if k_ is not None:
            _check(v_ is not None, "If key is supplied, value must also be passed in")
            _check(seqlens_k_ is not None, "If key is supplied, seqlens_k must also be passed in")
            _check(seqlen_q <= seqlen_k, "If key is supplied, it must have seqlen <= the seqlen of the KV cache")
            _check(k_.dtype == q_dtype, "Key must have the same dtype as query")
            _check(v_.dtype == q_dtype, "Value must have the same dtype as query")
            _check_device(k_, v_)
            _check(k_.stride(-1) == 1, "Key tensor must have contiguous last dimension")
            _check(v_.stride(-1) == 1, "Value tensor must have contiguous last dimension")
            seqlen_knew = k_.shape[1]
            _check(tuple(k_.shape) == (batch_size, seqlen_knew, num_heads_k, head_size_og), "k has the wrong shape")
            _check(tuple(v_.shape) == (batch_size, seqlen_knew, num_heads_k, head_size_og), "v has the wrong shape")
            k_padded, v_padded = _pad8(k_), _pad8(v_)
            keep += [k_padded, v_padded]
            p.seqlen_knew = seqlen_knew
            p.k_new, p.v_new = k_padded.data_ptr(), v_padded.data_ptr()
            p.knew_batch_stride, p.knew_row_stride, p.knew_head_stride = k_padded.stride(0), k_padded.stride(1), k_padded.stride(2)
            p.vnew_batch_stride, p.vnew_row_stride, p.vnew_head_stride = v_padded.stride(0), v_padded.stride(1), v_padded.stride(2)
        if seqlens_k_ is not None:
            _check(seqlens_k_.dtype == torch.int32, "seqlens_k must have dtype int32")
            _check_device(seqlens_k_)
            _check(seqlens_k_.is_contiguous(), "seqlens_k must be contiguous")
            _check(tuple(seqlens_k_.shape) == (batch_size,), "seqlens_k must have shape (batch_size)")
            p.cu_seqlens_k = seqlens_k_.data_ptr()
        p.is_seqlens_k_cumulative = int(seqlens_k_ is None)
        if rotary_cos_ is not None:
            _check(k_ is not None, "If rotary cos/sin are provided, new key / value to be appended to KV cache must also be provided")
            _check_device(rotary_cos_)
            rotary_dim = rotary_cos_.shape[1] * 2
            _check(rotary_dim <= head_size, "rotary_dim must be <= headdim")
            _check(rotary_dim % 16 == 0, "Only rotary dimensions divisible by 16 are currently supported")
            seqlen_ro = rotary_cos_.shape[0]
            _check(seqlen_ro >= seqlen_k, "cos/sin seqlen must be at least the seqlen of KV cache")
            _check(tuple(rotary_cos_.shape) == (seqlen_ro, rotary_dim // 2), "rotary_cos has the wrong shape")
            _check(rotary_cos_.is_contiguous(), "rotary_cos must be contiguous")
            _check(rotary_cos_.dtype == q_dtype, "rotary_cos must have the same dtype as query")
            _check(rotary_sin_ is not None, "If rotary cos is provided, rotary sin must also be provided")
            _check_device(rotary_sin_)
            _check(tuple(rotary_sin_.shape) == (seqlen_ro, rotary_dim // 2), "rotary_sin has the wrong shape")
            _check(rotary_sin_.is_contiguous(), "rotary_sin must be contiguous")
            _check(rotary_sin_.dtype == q_dtype, "rotary_cos must have the same dtype as query")
            p.rotary_cos, p.rotary_sin = rotary_cos_.data_ptr(), rotary_sin_.data_ptr()
            p.rotary_dim = rotary_dim
            p.is_rotary_interleaved = int(is_rotary_interleaved)
        if cache_batch_idx_ is not None:
            _check_device(cache_batch_idx_)
            _check(cache_batch_idx_.is_contiguous(), "cache_batch_idx must be contiguous")
            _check(cache_batch_idx_.dtype == torch.int32, "cache_batch_idx must have dtype int32")
            p.cache_batch_idx = cache_batch_idx_.data_ptr()
        _check(num_splits <= 128, "num_splits > 128 not supported")
        p.num_splits = max(int(num_splits), 0)
        if seqlen_q > 0 and seqlen_k > 0 and no_alloc:
            _call(lib.fa_fwd_kvcache_noalloc, p, _stream(q.device))
        elif seqlen_q > 0 and seqlen_k > 0:
            keep.append(_plan_and_alloc(p, 2, batch_size, num_heads, seqlen_q, head_size, q.device))
            _call(lib.fa_fwd_kvcache, p, _stream(q.device), q.device)
        else:
            out.zero_()
            softmax_lse.fill_(float("inf"))
        del keep

    if padded:
        out = out[..., :head_size_og]
        if out_ is not None:
            out_.copy_(out)
        if k_ is not None:
            # the appended rows live in the padded copies; write them back (flash_api.cpp:1263-1272)
            kcache.copy_(kcache_padded[..., :head_size_og])
            vcache.copy_(vcache_padded[..., :head_size_og])
    return [out, softmax_lse]


# FA_KERNEL_* of include/fa_mi355x.h
KERNEL_NAMES = {0: "none", 1: "tiled", 2: "tiled_tickets", 3: "pipelined", 4: "pingpong", 5: "wide", 6: "wide_pair",
                7: "decode", 8: "decode_tickets", 9: "pingpong_wide", 10: "pingpong_wide32"}


def last_kernel():
    """(name, dropout instantiation, key range split, head dims computed) of the attention kernel that the
    calling thread's last forward call launched: fa_last_kernel() decoded.  Host-side bookkeeping, no device
    work; tests assert with it that a case still reaches the kernel it was written for."""
    w = lib.fa_last_kernel()
    return KERNEL_NAMES.get(w & 0xff, "unknown"), bool(w & 0x100), bool(w & 0x200), (w >> 16) & 0xffff


def num_splits_heuristic_reference(batch_nheads_mblocks, num_sms, num_n_blocks, max_splits):
    return lib.fa_num_splits_heuristic_reference(batch_nheads_mblocks, num_sms, num_n_blocks, max_splits)
