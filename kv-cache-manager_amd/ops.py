"""Calls into libkvcm_hip.so.  Every function takes torch tensors that live on the GPU, checks on
the host that their shapes and dtypes are what the kernel assumes, and launches on torch's
current stream.  There is no fallback: without the library (or without a GPU) these raise.
"""
import ctypes as C
import os
import struct as _struct
import sys
import threading

import torch

from .csrc import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

_lock = threading.Lock()
_lib = None


class KernelError(RuntimeError):
    pass


def _declare(lib):
    vp, i, f = C.c_void_p, C.c_int, C.c_float

    def fn(name, *args):
        g = getattr(lib, name)
        g.restype = C.c_int
        g.argtypes = list(args)

    lib.kvcm_hip_last_error.restype = C.c_char_p
    fn("kvcm_embed", vp, vp, i, vp, i, i, i, vp)
    fn("kvcm_rmsnorm", vp, vp, i, vp, i, i, vp, vp, i, vp, i, i, i, f, i, vp)
    fn("kvcm_rope_cache", vp, i, i, vp, vp, vp, vp, vp, i, i, i, i, i, vp, i, vp, i, vp)
    fn("kvcm_rope_table", vp, vp, vp, i, i, vp)
    fn("kvcm_attention_decode_info", i, i, i, vp)
    fn("kvcm_attention_decode_fused_supported", i, i, i, i)
    fn("kvcm_attention_decode_fused", vp, i, vp, i, vp, vp, vp, vp, vp, i, vp, vp, i, i, i, i, i, f, vp, i, i, vp,
       C.c_longlong, vp)
    lib.kvcm_attention_decode_fused_scratch.restype = C.c_longlong
    lib.kvcm_attention_decode_fused_scratch.argtypes = [i, i, i, i, i]
    fn("kvcm_attention_generic_info", i, vp)
    fn("kvcm_attention_decode_fused_info", i, i, i, vp)
    fn("kvcm_gemm_skinny_swiglu_supported", i, i, i)
    fn("kvcm_gemm_skinny_swiglu", vp, vp, vp, i, i, i, i, i, i, i, vp)
    fn("kvcm_gemm_skinny_splits", i, i, i)
    fn("kvcm_gemm_skinny_waves", i, i, i, i, i)
    fn("kvcm_gemm_skinny_swiglu_normed_preferred", i, i, i)
    fn("kvcm_gemm_skinny_swiglu_normed", vp, vp, vp, i, f, vp, i, i, i, i, i, i, vp)
    fn("kvcm_gemm_skinny", vp, vp, vp, vp, i, i, i, i, i, i, i, i, vp)
    fn("kvcm_reduce_store", vp, vp, i, i, i, i, i, vp)
    fn("kvcm_swiglu", vp, vp, i, i, i, vp)
    fn("kvcm_add_residual", vp, vp, i, C.c_longlong, vp)
    fn("kvcm_gemm_f32", vp, vp, vp, i, i, i, i, i, i, vp)
    fn("kvcm_gemm_bf16", vp, vp, vp, i, i, i, i, i, i, i, vp)
    fn("kvcm_attention_generic", vp, i, i, vp, i, vp, vp, vp, i, vp, vp, i, i, i, i, i, f, i, vp)
    fn("kvcm_sample", vp, i, vp, vp, vp, vp, vp, i, i, vp)
    fn("kvcm_attention_decode_supported", i, i, i, i)
    fn("kvcm_attention_prefill_supported", i, i, i, i)
    fn("kvcm_attention_prefill", vp, i, vp, i, vp, vp, vp, i, vp, vp, i, i, i, i, i, i, i, i, f, vp, C.c_longlong, vp, vp)
    lib.kvcm_attention_prefill_scratch.restype = C.c_longlong
    lib.kvcm_attention_prefill_scratch.argtypes = [i, i, i, i, i, i]
    lib.kvcm_attention_prefill_segment.restype = i
    lib.kvcm_attention_prefill_segment.argtypes = [i, i, i, i, i, i]
    lib.kvcm_attention_prefill_tile_rows.restype = i
    lib.kvcm_attention_prefill_tile_rows.argtypes = [i, i, i, i, i, i]
    lib.kvcm_attention_decode_scratch.restype = C.c_longlong
    lib.kvcm_attention_decode_scratch.argtypes = [i, i, i, i]
    fn("kvcm_attention_decode", vp, i, vp, i, vp, vp, vp, i, vp, vp, i, i, i, i, i, f, i, vp, C.c_longlong, vp)
    fn("kvcm_gemm_library", vp, vp, vp, i, i, i, i, i, i, vp, C.c_longlong, vp)
    fn("kvcm_gemm_library_tuned", i, i, i, i, i, i)
    fn("kvcm_gemm_library_f32out_plan", i, i, i, i, i, i)
    fn("kvcm_gemm_library_f32out", vp, vp, vp, i, i, i, i, i, i, vp, C.c_longlong, vp)
    fn("kvcm_gemm_library_tune", vp, vp, i, C.c_longlong, vp, i, i, i, i, i, i, vp, C.c_longlong, vp, i, C.c_double,
       C.POINTER(C.c_double), vp)
    fn("kvcm_probe_empty", i, i, vp)
    fn("kvcm_probe_copy", vp, vp, C.c_longlong, i, vp)
    fn("kvcm_probe_read", vp, C.c_longlong, vp, i, vp)
    fn("kvcm_probe_stream", vp, C.c_longlong, vp, i, i, i, vp)
    fn("kvcm_probe_mfma", i, vp, i, vp)
    fn("kvcm_probe_barrier", vp, vp, vp, i, i, i, i, i, vp)
    fn("kvcm_probe_sums", vp, vp, vp, i, i, i, vp, vp)
    fn("kvcm_probe_phases", vp, C.POINTER(C.c_longlong), i, i, i, i, vp, vp, vp, vp, i, vp)
    fn("kvcm_fill_normal", vp, i, C.c_longlong, C.c_uint64, f, f, vp)
    fn("kvcm_fill_index", vp, C.c_longlong, C.c_uint64, i, vp)
    fn("kvcm_gemm8_supported", i, i, i)
    fn("kvcm_gemm8", vp, i, vp, i, i, i, i, vp, i, f, vp, i, i, i, vp)
    fn("kvcm_gemm8_residual_norm", vp, i, vp, i, i, i, i, vp, vp, i, vp, vp, vp)
    fn("kvcm_embed_scaled", vp, vp, i, vp, i, i, i, f, vp)
    fn("kvcm_gated_act", vp, i, vp, i, i, i, i, i, vp)
    fn("kvcm_rmsnorm_chain", vp, vp, i, vp, i, C.c_longlong, vp, vp, f, vp, vp, vp, vp, i, i, i, f, vp)
    fn("kvcm_head_norm_gate", vp, i, vp, i, vp, vp, i, i, i, i, i, f, vp)
    fn("kvcm_short_conv", vp, i, vp, vp, vp, vp, vp, i, i, vp, vp, vp, vp, vp, vp, i, i, i, i, i, vp)
    fn("kvcm_short_conv_state", vp, i, vp, vp, vp, vp, vp, vp, i, i, i, vp)
    fn("kvcm_rotary_pairs_table", vp, vp, i, i, f, vp)
    fn("kvcm_rotate_store", vp, i, vp, i, vp, i, i, vp, vp, i, i, vp, vp, i, i, i, i, i, i, vp)
    fn("kvcm_norm_rotate_store", vp, i, vp, vp, f, vp, i, f, vp, i, vp, i, i, vp, vp, i, i, vp, vp, i, i, i, i, i, i, vp)
    fn("kvcm_rotary_freq_table", vp, vp, vp, i, i, f, vp)
    fn("kvcm_dyt_norm", vp, i, vp, i, C.c_longlong, vp, vp, i, vp, vp, f, vp, vp, vp, f, vp, i, i, i, vp)
    fn("kvcm_stream_pack", vp, vp, vp, vp, vp, i, i, i, vp)
    fn("kvcm_scale_rows", vp, C.c_longlong, f, vp)
    fn("kvcm_softcap_rows", vp, C.c_longlong, f, vp)
    fn("kvcm_head_gate", vp, i, i, vp, i, i, i, i, i, vp)
    fn("kvcm_rms_groups", vp, i, i, i, i, vp, f, vp, i, i, i, vp)
    fn("kvcm_layernorm_post", vp, vp, i, C.c_longlong, vp, f, vp, vp, vp, i, i, i, f, vp)
    fn("kvcm_head_norm_store", vp, i, vp, vp, vp, f, vp, f, i, i, vp, vp, i, i, vp, vp, i, i, i, i, i, i, vp)
    fn("kvcm_gemm_heads", vp, i, i, vp, vp, i, i, vp, i, i, i, i, i, vp)
    fn("kvcm_act_rows", vp, i, i, C.c_longlong, vp, i, i, i, i, i, vp)
    fn("kvcm_mlstm_scan", vp, i, vp, i, vp, i, vp, i, vp, i, vp, vp, f, f, vp, vp, vp, i, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, vp)
    fn("kvcm_moe_route", vp, i, i, C.c_longlong, i, i, i, vp, vp, i, vp)
    fn("kvcm_moe_table_route", vp, vp, i, i, i, vp, vp, i, vp)
    fn("kvcm_moe_up", vp, i, i, vp, vp, vp, i, i, i, i, i, i, vp)
    fn("kvcm_moe_down", vp, i, vp, vp, vp, vp, vp, i, i, i, i, i, vp)
    fn("kvcm_moe_grouped_supported", i, i, i)
    fn("kvcm_moe_grouped_max_tiles", i, i)
    fn("kvcm_moe_grouped", vp, i, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, vp)
    fn("kvcm_pool_update", vp, vp, i, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, i, vp)
    fn("kvcm_attention_window_pool", vp, i, i, vp, i, vp, vp, vp, vp, vp, i, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, f, i, i, i, i, f, vp)
    fn("kvcm_attention_window_pool_tiles_supported", i, i, i)
    fn("kvcm_attention_window_pool_tiles", vp, i, vp, i, vp, vp, vp, vp, vp, i, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, i, f, i, i, i, i, f, vp)
    fn("kvcm_selective_scan", vp, i, i, vp, i, vp, vp, i, i, i, vp, vp, vp, i, vp, i, vp, vp, vp, vp, i, i, i, i, i, i, vp, C.c_longlong, i, vp)
    fn("kvcm_scan_prepare", vp, i, vp, vp, i, i, i, vp)
    fn("kvcm_delta_prepare", vp, i, vp, i, vp, vp, i, vp, i, vp, vp, vp, vp, i, i, i, vp)
    fn("kvcm_delta_scan", vp, i, vp, i, vp, i, vp, vp, vp, vp, i, vp, vp, vp, vp, i, i, i, i, vp)
    lib.kvcm_gemm_library_workspace_bytes.restype = C.c_longlong
    lib.kvcm_gemm_library_workspace_bytes.argtypes = []
    lib.kvcm_program_new.restype = vp
    lib.kvcm_program_new.argtypes = []
    lib.kvcm_program_delete.restype = None
    lib.kvcm_program_delete.argtypes = [vp]
    fn("kvcm_program_add", vp, C.c_char_p, C.POINTER(C.c_uint64), i)
    fn("kvcm_program_size", vp)
    fn("kvcm_program_run", vp, vp)
    lib.kvcm_engine_new.restype = vp
    lib.kvcm_engine_new.argtypes = [vp, C.POINTER(C.c_uint64), vp, vp, C.c_longlong, vp, vp, i, i, i, i, i, i, i, i, vp]
    lib.kvcm_engine_delete.restype = None
    lib.kvcm_engine_delete.argtypes = [vp]
    fn("kvcm_engine_plan", vp, C.c_double, C.POINTER(C.c_int64))
    fn("kvcm_engine_last_plan", vp, C.POINTER(C.c_int64))
    fn("kvcm_engine_register", vp, vp, i)
    fn("kvcm_engine_run", vp, C.c_double, i, C.POINTER(C.c_int64))
    fn("kvcm_engine_add", vp, C.c_longlong, C.POINTER(C.c_int32), i, i, f, C.c_uint64, C.c_double)
    fn("kvcm_engine_idle", vp)
    fn("kvcm_engine_step", vp, C.c_double, C.POINTER(C.c_int64))
    fn("kvcm_engine_take_finished", vp)
    fn("kvcm_engine_finished_get", vp, i, C.POINTER(C.c_int64), C.POINTER(C.c_double), C.POINTER(C.c_int32), i)
    lib.kvcm_engine_finished_clear.restype = None
    lib.kvcm_engine_finished_clear.argtypes = [vp]
    lib.kvcm_engine_stats.restype = None
    lib.kvcm_engine_stats.argtypes = [vp, C.POINTER(C.c_int64)]


def lib():
    global _lib
    with _lock:
        if _lib is None:
            loaded = C.CDLL(_build.build_hip())
            _declare(loaded)
            _lib = loaded
    return _lib


def library_path():
    lib()
    return _lib._name


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream's handle (of device 0: the engine runs on one GPU).  The raw getter
    costs a fraction of a microsecond; building a Stream object costs several, on every launch."""
    if _raw_stream is not None:
        return _raw_stream(0)
    return torch.cuda.current_stream().cuda_stream


def _check(rc):
    if rc != 0:
        raise KernelError(lib().kvcm_hip_last_error().decode())


# ------------------------------------------------------------------------------ recorded steps
class StepProgram:
    """The launches of one step, kept natively (csrc/hip/step_program.hip): every launching entry that
    is called while a program records is appended to it with its arguments, and ``run`` calls the same
    entries again without Python.  Whoever registers the program with the native engine hands its
    ownership over (``release``)."""

    def __init__(self):
        self._h = lib().kvcm_program_new()

    def __len__(self):
        return lib().kvcm_program_size(self._h)

    def add(self, name, slots):
        arr = (C.c_uint64 * len(slots))(*slots)
        _check(lib().kvcm_program_add(self._h, name.encode(), arr, len(slots)))

    def run(self, stream=None):
        _check(lib().kvcm_program_run(self._h, _stream() if stream is None else stream))

    def release(self):
        h, self._h = self._h, None
        return h

    def __del__(self):
        if getattr(self, "_h", None):
            lib().kvcm_program_delete(self._h)
            self._h = None


_recording = None      # the StepProgram that launches are appended to, while one records
_MASK64 = (1 << 64) - 1


class recording:
    """``with ops.recording(program): ...``: every launch inside also goes into ``program``.  Anything a
    step does that is not a launching entry of this library (a tensor library's routine, an allocation)
    would be missing from the replay: parts that do such things are not capturable."""

    def __init__(self, program):
        self.program = program

    def __enter__(self):
        global _recording
        if _recording is not None:
            raise RuntimeError("a step program is already recording")
        _recording = self.program
        return self.program

    def __exit__(self, *exc):
        global _recording
        _recording = None
        return False


def _slots(fn, args):
    out = []
    for t, a in zip(fn.argtypes, args):
        if t is C.c_float:
            out.append(_struct.unpack("<I", _struct.pack("<f", a))[0])
        elif a is None:
            out.append(0)
        else:
            out.append(int(a) & _MASK64)
    return out


# KVCM_SYNC_LAUNCHES=1: every launching entry is named on stderr before it is called and waited for after it, so that a
# kernel's failure is reported at its own call (for hunting faults; steps run many times slower).
_SYNC_LAUNCHES = bool(int(os.environ.get("KVCM_SYNC_LAUNCHES", "0") or 0))


def _call(name, *args):
    """Calls a launching entry; while a program records, notes the call there first."""
    fn = getattr(lib(), name)
    if _recording is not None:
        _recording.add(name, _slots(fn, args))
    if _SYNC_LAUNCHES:
        print("[kvcm launch] %s %s" % (name, " ".join(str(a) for a in args if isinstance(a, (int, float)) and abs(a) < 1 << 20)),
              file=sys.stderr, flush=True)
        _check(fn(*args))
        torch.cuda.synchronize()
        return
    _check(fn(*args))


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _dev(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernel operands must live on the GPU")


def _i32(t, name, n=None):
    if t is None:
        return
    _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be a contiguous int32 tensor")
    if n is not None:
        _need(t.numel() >= n, f"{name} holds {t.numel()} entries, {n} are needed")


def _rows2d(t, name):
    _need(t.dim() == 2 and t.stride(1) == 1, f"{name} must be 2-d with unit inner stride")


# --------------------------------------------------------------------------------------------
def embed(ids, table, out):
    """out[t, :] = float(table[ids[t], :]);  out is the 32-bit residual stream [T, H]."""
    _dev(ids, table, out)
    T, H = out.shape
    _i32(ids, "ids", T)
    _need(table.dim() == 2 and table.shape[1] == H and table.is_contiguous(), "embedding table must be [V, H]")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "residual stream must be contiguous float32")
    _call("kvcm_embed", _ptr(ids), _ptr(table), _DT[table.dtype], _ptr(out), T, H, table.shape[0], _stream())


class PartialSums:
    """The output of a split-K product that has not been added up yet: ``data`` holds [splits, rows,
    cols] 32-bit sums.  The fused consumers (rmsnorm's ``add``, rope_cache's ``source``) add them in
    split order and round the sum to ``dtype`` as the stored product would have been."""

    def __init__(self, data, splits, rows, cols, out):
        self.data, self.splits, self.rows, self.cols, self.out = data, splits, rows, cols, out
        self.dtype = out.dtype

    def materialize(self):
        """Adds the splits up into the product's own output buffer [rows, cols] and returns it."""
        _call("kvcm_reduce_store", _ptr(self.data), _ptr(self.out), _DT[self.out.dtype], self.rows, self.cols,
                                       self.out.stride(0), self.splits, _stream())
        return self.out


# Decode steps of at most this many rows may fold their RMS norms into the products around them
# (csrc/hip/gemm_rows8.hip); how many rows of that a model's steps do fold is the engine's to say
# (StepView.fold_rows).
FUSED_NORM_MAX_ROWS = 8


def gemm8_supported(M, N, K):
    return bool(lib().kvcm_gemm8_supported(M, N, K))


class PendingProduct:
    """A product x @ w^T that has not run yet, handed on so that whoever adds it to the residual
    stream can choose how it runs: with the addition and the following norm's preparation in its
    epilogue (``gemm_residual_norm``), or the ordinary way (``run``).  ``out`` and ``scratch`` are the
    buffers the ordinary way uses."""

    def __init__(self, x, w, out, scratch=None):
        self.x, self.w, self.out, self.scratch = x, w, out, scratch
        self.dtype = out.dtype

    def run(self, keep_partial=False):
        return gemm(self.x, self.w, self.out, scratch=self.scratch, keep_partial=keep_partial)

    def materialize(self):
        return self.run(False)


class NormedRows:
    """The rows a product after an RMS norm multiplies, with the norm's scale still to be applied:
    ``xg`` = round(g * round(x)) [rows, H] and ``ss`` [rows, H / 8] sums of x^2 per 8-column tile, left
    by ``gemm_residual_norm``.  ``gemm`` and ``gemm_swiglu`` take it in x's place and scale their sums
    by rsqrt(mean x^2 + eps); ``materialize`` gives the ordinary normed rows instead (the residual
    stream x already holds the addition)."""

    def __init__(self, xg, ss, eps, x, weight, out):
        self.xg, self.ss, self.eps, self.x, self.weight, self.out = xg, ss, float(eps), x, weight, out
        self.shape, self.dtype = xg.shape, xg.dtype

    def materialize(self):
        rmsnorm(self.x, self.weight, self.out, self.eps)
        return self.out


def gemm_residual_norm(product, x, weight, eps, xg, ss, out):
    """x += round(product); returns NormedRows for the norm (weight, eps) that follows: the producer
    half of the folded norm.  product: PendingProduct of at most 8 bfloat16 rows; x: the 32-bit residual
    stream [rows, H]; xg [>= rows, H] bfloat16 and ss [>= rows, H / 8] float32 receive the result; out:
    where ``materialize`` would put ordinary normed rows."""
    a, w = product.x, product.w
    M, K = a.shape
    H = w.shape[0]
    _dev(a, w, x, weight, xg, ss)
    _rows2d(a, "x")
    _rows2d(w, "w")
    _need(a.dtype == w.dtype == torch.bfloat16 and w.shape[1] == K, "gemm_residual_norm needs bfloat16 operands [M, K], [H, K]")
    _need(x.dtype == torch.float32 and x.is_contiguous() and tuple(x.shape) == (M, H), "the residual stream must be contiguous float32 [M, H]")
    _need(weight.numel() == H and weight.is_contiguous(), "norm weight must have H entries")
    _need(xg.dtype == torch.bfloat16 and xg.is_contiguous() and xg.shape[0] >= M and xg.shape[1] == H, "xg must be bfloat16 [>= M, H]")
    _need(ss.dtype == torch.float32 and ss.is_contiguous() and ss.shape[0] >= M and ss.shape[1] == H // 8 and H % 8 == 0,
          "ss must be float32 [>= M, H / 8]")
    _call("kvcm_gemm8_residual_norm", _ptr(a), a.stride(0), _ptr(w), w.stride(0), M, H, K, _ptr(x), _ptr(weight),
          _DT[weight.dtype], _ptr(xg), _ptr(ss), _stream())
    return NormedRows(xg[:M], ss[:M], eps, x, weight, out)


def _gemm8(x, w, out, N, swiglu):
    """The product of at most 8 rows (gemm_rows8.hip); x: a tensor or NormedRows."""
    normed = isinstance(x, NormedRows)
    a = x.xg if normed else x
    M, K = a.shape
    _call("kvcm_gemm8", _ptr(a), a.stride(0), _ptr(w), w.stride(0), M, N, K, _ptr(x.ss) if normed else 0,
          x.ss.shape[1] if normed else 0, x.eps if normed else 0.0, _ptr(out), _DT[out.dtype], out.stride(0), int(swiglu),
          _stream())


def rmsnorm(x, weight, out, eps, add=None, rows=None, write_back=True):
    """v = x[src] (+ add[src]); x[src] = v when write_back; out[r] = weight * round(v * rsqrt(mean v^2 + eps)).
    src = rows[r] if rows is given, else r.  ``add`` is a tensor of x's shape or PartialSums."""
    partial = add if isinstance(add, PartialSums) else None
    if partial is not None:
        _need(partial.cols == x.shape[1] and partial.rows == x.shape[0], "partial sums must match x")
        add = None
    _dev(x, weight, out, add, rows)
    R, H = out.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == H, "x must be contiguous float32 [T, H]")
    _need(weight.numel() == H and weight.is_contiguous(), "norm weight must have H entries")
    _need(out.is_contiguous(), "norm output must be contiguous")
    if rows is None:
        _need(x.shape[0] >= R, "x has fewer rows than the output")
    else:
        _i32(rows, "rows", R)
    if add is not None:
        _need(add.shape == x.shape and add.is_contiguous(), "add must match x")
    wb = bool(write_back) and (add is not None or partial is not None) and rows is None
    _call("kvcm_rmsnorm", _ptr(x), _ptr(add), _DT[add.dtype] if add is not None else 0,
                              _ptr(partial.data) if partial else 0, partial.splits if partial else 0,
                              partial.rows if partial else 0, _ptr(rows), _ptr(weight),
                              _DT[weight.dtype], _ptr(out), _DT[out.dtype], R, H, float(eps), int(wb), _stream())


def rope_table(positions, inv_freq, out, rows=None):
    """out[t, j] = (cos, sin) of float(positions[t]) * inv_freq[j]: the angles of a step, computed
    once and read by every layer's rotation."""
    _dev(positions, inv_freq, out)
    T = out.shape[0] if rows is None else rows
    _i32(positions, "positions", T)
    _need(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "inv_freq must be float32")
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.dim() == 3 and out.shape[1] == inv_freq.numel()
          and out.shape[2] == 2 and out.shape[0] >= T, "the table must be float32 [rows, head_dim/2, 2]")
    _call("kvcm_rope_table", _ptr(positions), _ptr(inv_freq), _ptr(out), T, inv_freq.numel(), _stream())
    return out


def rope_cache(qkv, nh, nkv, hd, positions=None, inv_freq=None, slots=None, kcache=None, vcache=None,
               block_size=0, rows=None, source=None, cos_sin=None, skip_q=False):
    """Rotates the q and k heads of the fused rows in place (by the angles position * inv_freq, or
    by a table ``cos_sin`` [rows, hd/2, 2] computed beforehand; neither: no rotation) and copies k
    (rotated) and v to the paged cache (slots given).  Keys [pages, nkv, block_size, hd], values
    [pages, nkv, hd, block_size].  With ``source`` (PartialSums of the projection) the rows are read
    from there; q lands in ``qkv``.  ``skip_q``: the q heads are left as they are (``attention_prefill``
    rotates them as it reads them when it is given the same table)."""
    _dev(qkv, positions, inv_freq, slots, kcache, vcache)
    _rows2d(qkv, "qkv")
    T = qkv.shape[0] if rows is None else rows
    if source is not None:
        _need(isinstance(source, PartialSums) and source.rows == T and source.cols == (nh + 2 * nkv) * hd,
              "the partial sums do not have the shape of the fused rows")
    _need(qkv.shape[1] >= (nh + 2 * nkv) * hd, "qkv rows are too short for the head layout")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == hd // 2 and inv_freq.is_contiguous(),
              "inv_freq must hold head_dim/2 float32 values")
        if cos_sin is None:
            _need(positions is not None, "rotation needs positions")
            _i32(positions, "positions", T)
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.numel() >= T * hd
              and cos_sin.is_cuda, "cos_sin must be float32 [rows, head_dim/2, 2]")
    if slots is not None:
        _i32(slots, "slots", T)
        _need(kcache is not None and kcache.dtype == qkv.dtype and kcache.is_contiguous() and kcache.dim() == 4
              and tuple(kcache.shape[1:]) == (nkv, block_size, hd), "key cache must be [pages, nkv, block_size, hd]")
        _need(vcache is not None and vcache.dtype == qkv.dtype and vcache.is_contiguous() and vcache.dim() == 4
              and tuple(vcache.shape[1:]) == (nkv, hd, block_size), "value cache must be [pages, nkv, hd, block_size]")
    _call("kvcm_rope_cache", _ptr(qkv), _DT[qkv.dtype], qkv.stride(0), _ptr(positions), _ptr(inv_freq),
                                 _ptr(slots), _ptr(kcache), _ptr(vcache), T, nh, nkv, hd, block_size,
                                 _ptr(source.data) if source is not None else 0,
                                 source.splits if source is not None else 0, _ptr(cos_sin), 1 if skip_q else 0, _stream())


def swiglu(gate_up, out):
    _dev(gate_up, out)
    T, I = out.shape
    _need(gate_up.shape == (T, 2 * I) and gate_up.is_contiguous() and out.is_contiguous()
          and gate_up.dtype == out.dtype, "swiglu needs [T, 2I] -> [T, I] of one dtype")
    _call("kvcm_swiglu", _ptr(gate_up), _ptr(out), _DT[out.dtype], T, I, _stream())


def add_residual(x, y):
    _dev(x, y)
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.shape == y.shape,
          "add_residual needs a float32 x and a y of the same shape")
    _call("kvcm_add_residual", _ptr(x), _ptr(y), _DT[y.dtype], x.numel(), _stream())


# Rows from which a bfloat16 product is handed to the library (hipBLASLt, called directly:
# csrc/hip/gemm_library.hip); the reference leaves every product to its vendor library.  0 = always
# use the kernels of this package.  Below, the weight-streaming kernels of this package run.  Measured
# end to end at TinyLlama sizes (steps of 16 decoding rows beside a prompt portion, replayed from
# recorded programs, so that a call costs the host the same either way): 48 rows 2.03 ms with this
# package's kernels against 2.24 with the library's, 80 rows 2.05 / 2.26, 112 rows 2.83 / 2.61,
# 176 rows 2.85 / 2.56, 336 rows 3.85 / 2.98.
LIBRARY_GEMM_MIN_ROWS = 96
# ... except that up to LIBRARY_LONG_K_MIN_ROWS - 1 rows this package's kernel keeps the products whose K is
# at least their width and whose weights are at least LIBRARY_LONG_K_BYTES (the O and down projections of 7B /
# 8B sizes): the library's first choice is slow there.  Measured at Llama-3-8B sizes, library against this
# package's kernel: down 74.9 / 44.3 us at 128 rows, 102 / 69 at 192, 61.5 / 72.5 at 256; O 23.1 / 19.3 at 128,
# 31.9 / 26.6 at 192, 21.9 / 28.6 at 256; a prompt step of 128 rows 7.15 -> 6.38 ms.  TinyLlama's down projection
# (23 MB) is the library's at every row count from 96 on (12.9 / 16.4 us at 128 rows).
LIBRARY_LONG_K_MIN_ROWS = 193
LIBRARY_LONG_K_BYTES = 32 << 20


def _library_takes(M, N, K):
    """Does a bfloat16 product of M rows go to the vendor library?"""
    if not LIBRARY_GEMM_MIN_ROWS or M < LIBRARY_GEMM_MIN_ROWS:
        return False
    return not (M < LIBRARY_LONG_K_MIN_ROWS and K >= N and 2 * N * K >= LIBRARY_LONG_K_BYTES)


# Which of the library's algorithms a shape runs.  "off": the first choice of the library's heuristic.
# "heuristic": at a shape's first use the heuristic's choices (up to 16) are timed on the call's own
# operands and the fastest is kept: some 400 launches of the product, 20 to 40 milliseconds per shape, for
# about 5 % of its time afterwards, which pays after thousands of calls of that shape.  "all": every
# algorithm of the library that supports the shape is timed (seconds per shape, at most
# LIBRARY_TUNING_SECONDS).  Off unless the engine's configuration asks for it: a serving run meets a few
# hundred shapes (rows in steps of 64, four products) and most of them only a few times; measured on a
# burst of 400 requests, tuning each at its first use took longer than the whole run without it.
LIBRARY_TUNING = "off"
LIBRARY_TUNING_SECONDS = 6.0
LIBRARY_TUNING_BYTES = 512 << 20
_TUNING_MODES = {"off": 0, "heuristic": 1, "all": 2}
library_tuning_log = []          # (M, N, K, first choice's us, kept us, candidates timed) per tuned shape

_library_ws = None


_f32out_shapes = {}


def _library_has_f32out(*shape):
    """Does the library have an algorithm for this product with a 32-bit result?  Asked once per shape (the plan is
    made then, outside any recorded launch)."""
    if shape not in _f32out_shapes:
        _f32out_shapes[shape] = lib().kvcm_gemm_library_f32out_plan(*shape) == 0
    return _f32out_shapes[shape]


def _library_workspace(device):
    """Device memory the vendor library's product may use (one buffer, kept: recorded steps hold its address)."""
    global _library_ws
    if _library_ws is None:
        _library_ws = torch.empty(lib().kvcm_gemm_library_workspace_bytes(), dtype=torch.uint8, device=device)
    return _library_ws


def skinny_waves(M, N, K, S=1, swiglu=False):
    """Waves per workgroup the shared-rows kernel runs this bfloat16 product with (0: another kernel takes it)."""
    return lib().kvcm_gemm_skinny_waves(int(M), int(N), int(K), int(S), int(bool(swiglu)))


def skinny_splits(M, N, K):
    """Split count the decode-shaped kernel uses for this shape, 0 when it does not take it."""
    return lib().kvcm_gemm_skinny_splits(M, N, K)


def gemm(x, w, out, scratch=None, keep_partial=False, tuning=None):
    """out[M, N] = x[M, K] @ w[N, K]^T.  float32 x float32 -> float32 (plain FMA, fixed k order), or
    bfloat16 x bfloat16 -> bfloat16 | float32 (MFMA, 32-bit accumulation).

    Rows below LIBRARY_GEMM_MIN_ROWS take the weight-streaming kernels (also more rows, up to 512,
    while the library is switched off: inside a captured graph); when they split K they need
    ``scratch`` (float32, at least splits*M*N elements).  With ``keep_partial``
    the un-added partial sums are returned as PartialSums (for a fused consumer) instead of ``out``.
    ``tuning``: which of the library's algorithms a many-row product runs ("off" | "heuristic" | "all";
    None: this module's LIBRARY_TUNING); an engine passes its own option, so that two engines in one
    process do not change each other's.
    """
    if isinstance(x, NormedRows):
        M, K = x.shape
        N = w.shape[0]
        _dev(x.xg, x.ss, w, out)
        _rows2d(w, "w")
        _rows2d(out, "out")
        if (w.dtype == torch.bfloat16 and w.shape[1] == K and out.shape == (M, N) and gemm8_supported(M, N, K)
                and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0):
            _gemm8(x, w, out, N, False)
            return out
        x = x.materialize()
    _dev(x, w, out)
    for t, n in ((x, "x"), (w, "w"), (out, "out")):
        _rows2d(t, n)
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K and out.shape == (M, N), f"gemm shapes do not agree: {tuple(x.shape)} {tuple(w.shape)} {tuple(out.shape)}")
    if x.dtype == torch.float32:
        _need(w.dtype == torch.float32 and out.dtype == torch.float32, "a float32 gemm needs float32 operands")
        _call("kvcm_gemm_f32", _ptr(x), _ptr(w), _ptr(out), M, N, K, x.stride(0), w.stride(0), out.stride(0), _stream())
        return out
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm operands must both be bfloat16")
    if out.dtype == torch.float32 and out.is_contiguous() and _library_takes(M, N, K) and _library_has_f32out(
            M, N, K, x.stride(0), w.stride(0), out.stride(0)):
        # many rows, a 32-bit result: the library stores its 32-bit sums as they are
        ws = _library_workspace(out.device)
        _call("kvcm_gemm_library_f32out", _ptr(x), _ptr(w), _ptr(out), M, N, K, x.stride(0), w.stride(0), out.stride(0),
              _ptr(ws), ws.numel(), _stream())
        return out
    library = _library_takes(M, N, K) and out.dtype == torch.bfloat16 and out.is_contiguous()
    S = skinny_splits(M, N, K) if (not library and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
                                   and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0) else 0
    if S > 1 and (scratch is None or scratch.numel() < S * M * N):
        S = 1 if scratch is None else max(1, min(S, scratch.numel() // (M * N)))
    if S >= 1:
        if S > 1:
            _need(scratch.dtype == torch.float32 and scratch.is_contiguous() and scratch.is_cuda, "scratch must be float32")
        _call("kvcm_gemm_skinny", _ptr(x), _ptr(w), _ptr(scratch) if S > 1 else 0, _ptr(out), _DT[out.dtype], M, N, K,
                                      x.stride(0), w.stride(0), out.stride(0), S, _stream())
        if S == 1:
            return out
        partial = PartialSums(scratch, S, M, N, out)
        return partial if keep_partial else partial.materialize()
    if library:
        ws = _library_workspace(out.device)
        mode = _TUNING_MODES[LIBRARY_TUNING if tuning is None else tuning]
        shape = (M, N, K, x.stride(0), w.stride(0), out.stride(0))
        if mode and lib().kvcm_gemm_library_tuned(*shape) < mode:
            # not a recorded launch: it runs here, once, whoever is recording
            check = torch.empty(M * N + 4, dtype=torch.bfloat16, device=out.device)
            # copies of the weights that timed calls go round, about LIBRARY_TUNING_BYTES in all: a model's layers
            # bring theirs from memory, not from a cache that one matrix alone would stay in
            span = (N - 1) * w.stride(0) + K
            copies = max(1, min(16, LIBRARY_TUNING_BYTES // (2 * span)))
            rows = torch.empty(copies, span, dtype=torch.bfloat16, device=out.device)
            rows.copy_(torch.as_strided(w, (span,), (1,)).unsqueeze(0).expand(copies, span))
            report = (C.c_double * 3)()
            rc = lib().kvcm_gemm_library_tune(_ptr(x), _ptr(rows), copies, 2 * span, _ptr(out), *shape, _ptr(ws), ws.numel(),
                                              _ptr(check), mode, float(LIBRARY_TUNING_SECONDS), report, _stream())
            del rows, check
            if rc != 0:
                raise KernelError(lib().kvcm_hip_last_error().decode())
            library_tuning_log.append((M, N, K, report[0], report[1], int(report[2])))
        _call("kvcm_gemm_library", _ptr(x), _ptr(w), _ptr(out), M, N, K, x.stride(0), w.stride(0), out.stride(0),
              _ptr(ws), ws.numel(), _stream())
        return out
    _call("kvcm_gemm_bf16", _ptr(x), _ptr(w), _ptr(out), _DT[out.dtype], M, N, K, x.stride(0), w.stride(0),
                                out.stride(0), _stream())
    return out


def gemm_swiglu(x, w_gate_up, out):
    """out[M, I] = swiglu(x[M, K] @ w_gate_up[2 I, K]^T) in one launch, or False when this shape
    has no fused kernel (then the caller runs the product and ``swiglu`` one after the other:
    the same values up to the order of the sums)."""
    if isinstance(x, NormedRows):
        M, K = x.shape
        I = out.shape[1]
        _dev(x.xg, x.ss, w_gate_up, out)
        _rows2d(w_gate_up, "w_gate_up")
        _rows2d(out, "out")
        if not (w_gate_up.dtype == out.dtype == torch.bfloat16 and tuple(w_gate_up.shape) == (2 * I, K) and out.shape[0] == M
                and gemm8_supported(M, I, K) and w_gate_up.stride(0) % 8 == 0 and w_gate_up.data_ptr() % 16 == 0):
            return False          # the caller materializes the rows and comes again
        if lib().kvcm_gemm_skinny_swiglu_normed_preferred(M, I, K) and x.xg.stride(0) % 8 == 0:
            _call("kvcm_gemm_skinny_swiglu_normed", _ptr(x.xg), _ptr(w_gate_up), _ptr(x.ss), x.ss.shape[1], x.eps, _ptr(out),
                  M, I, K, x.xg.stride(0), w_gate_up.stride(0), out.stride(0), _stream())
        else:
            _gemm8(x, w_gate_up, out, I, True)
        return True
    _dev(x, w_gate_up, out)
    for t, n in ((x, "x"), (w_gate_up, "w_gate_up"), (out, "out")):
        _rows2d(t, n)
    M, K = x.shape
    I = out.shape[1]
    _need(w_gate_up.shape == (2 * I, K) and out.shape[0] == M, "gemm_swiglu shapes do not agree")
    if LIBRARY_GEMM_MIN_ROWS and M >= LIBRARY_GEMM_MIN_ROWS:
        return False          # many rows: the library product, then swiglu
    if not (x.dtype == w_gate_up.dtype == out.dtype == torch.bfloat16 and x.stride(0) % 8 == 0
            and w_gate_up.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0
            and lib().kvcm_gemm_skinny_swiglu_supported(M, I, K)):
        return False
    _call("kvcm_gemm_skinny_swiglu", _ptr(x), _ptr(w_gate_up), _ptr(out), _DT[out.dtype], M, I, K, x.stride(0),
                                         w_gate_up.stride(0), out.stride(0), _stream())
    return True


def _check_caches(kcache, vcache, nkv, hd, packed_offsets=False):
    _need(kcache.dim() == 4 and kcache.is_contiguous() and kcache.shape[1] == nkv and kcache.shape[3] == hd,
          "key cache must be [pages, nkv, block_size, hd]")
    _need(vcache.dim() == 4 and vcache.is_contiguous() and tuple(vcache.shape) == (kcache.shape[0], nkv, hd, kcache.shape[2]),
          "value cache must be [pages, nkv, hd, block_size]")
    _need(kcache.shape[0] * kcache.shape[2] < 2 ** 31, "a cache of 2^31 token slots or more does not fit 32-bit slot numbers")
    # the decode kernels keep a token's offset inside one layer's cache as 32 bits in units of 8 elements
    _need(not packed_offsets or kcache.numel() <= 2 ** 35,
          "one layer's key cache beyond 2^35 elements (64 GiB of bfloat16) does not fit the decode kernels' page offsets")


def attention(q, out, kcache, vcache, tables, table_stride, row_seq, ctx_lens, nh, nkv, hd, scale, window=0,
              rows=None):
    """out[r, h, :] = softmax(scale * q[r, h] . K[0:ctx_r]) V[0:ctx_r] over the paged cache."""
    _dev(q, out, kcache, vcache, tables, row_seq, ctx_lens)
    _rows2d(q, "q")
    _rows2d(out, "out")
    T = q.shape[0] if rows is None else rows
    _need(q.dtype == out.dtype == kcache.dtype == vcache.dtype, "attention operands must share one dtype")
    _check_caches(kcache, vcache, nkv, hd)
    _i32(row_seq, "row_seq", T)
    _i32(ctx_lens, "ctx_lens", T)
    _i32(tables, "tables")
    _call("kvcm_attention_generic", _ptr(q), _DT[q.dtype], q.stride(0), _ptr(out), out.stride(0), _ptr(kcache),
                                        _ptr(vcache), _ptr(tables), table_stride, _ptr(row_seq), _ptr(ctx_lens), T, nh,
                                        nkv, hd, kcache.shape[2], float(scale), int(window), _stream())


def attention_decode_supported(nh, nkv, hd, dtype, block_size=16):
    return dtype == torch.bfloat16 and bool(lib().kvcm_attention_decode_supported(nh, nkv, hd, block_size))


def attention_kernel_info(variant, nh, nkv, hd):
    """{"regs", "lds_bytes", "workgroups_per_cu", "threads"} of the compiled bfloat16 attention
    kernel: variant "v1" (one pass per row and head), "v2" (partitioned) or "fused" (one launch
    with rotation and page write)."""
    out = (C.c_int * 4)()
    if variant == "v1":
        _check(lib().kvcm_attention_generic_info(hd, out))
    elif variant == "fused":
        _check(lib().kvcm_attention_decode_fused_info(nh, nkv, hd, out))
    else:
        _check(lib().kvcm_attention_decode_info(nh, nkv, hd, out))
    return dict(regs=out[0], lds_bytes=out[1], workgroups_per_cu=out[2], threads=out[3])


def attention_decode_scratch(rows, nh, hd, max_context):
    return int(lib().kvcm_attention_decode_scratch(rows, nh, hd, max_context))


def attention_decode(q, out, kcache, vcache, tables, table_stride, row_seq, ctx_lens, nh, nkv, hd, scale, max_context,
                     scratch, rows=None):
    """The same result as ``attention`` for bfloat16, contexts cut into partitions of 256 tokens
    that run in parallel and are merged; ``max_context`` bounds every row's context length."""
    _dev(q, out, kcache, vcache, tables, row_seq, ctx_lens, scratch)
    _rows2d(q, "q")
    _rows2d(out, "out")
    T = q.shape[0] if rows is None else rows
    _need(q.dtype == out.dtype == kcache.dtype == vcache.dtype == torch.bfloat16, "attention_decode is bfloat16 only")
    _check_caches(kcache, vcache, nkv, hd, packed_offsets=True)
    _need(scratch.dtype == torch.float32 and scratch.is_contiguous(), "scratch must be contiguous float32")
    _i32(row_seq, "row_seq", T)
    _i32(ctx_lens, "ctx_lens", T)
    _i32(tables, "tables")
    _call("kvcm_attention_decode", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(kcache), _ptr(vcache),
                                       _ptr(tables), table_stride, _ptr(row_seq), _ptr(ctx_lens), T, nh, nkv, hd,
                                       kcache.shape[2], float(scale), int(max_context), _ptr(scratch), scratch.numel(),
                                       _stream())


def attention_decode_fused_supported(nh, nkv, hd, dtype, block_size=16):
    return dtype == torch.bfloat16 and bool(lib().kvcm_attention_decode_fused_supported(nh, nkv, hd, block_size))


def attention_decode_fused_scratch(rows, nh, nkv, hd, max_context):
    """Floats of scratch ``attention_decode_fused`` needs for these sizes (0: contexts are not cut
    into parts: short ones, or rows x kv heads fill the chip)."""
    return int(lib().kvcm_attention_decode_fused_scratch(rows, nh, nkv, hd, max_context))


def attention_decode_fused(projection, out, kcache, vcache, tables, table_stride, row_seq, ctx_lens, nh, nkv, hd, scale,
                           cos_sin=None, slots=None, rows=None, max_context=0, scratch=None):
    """From the QKV projection to the attention output for rows of different sequences (bfloat16):
    ``projection`` is the fused [q | k | v] rows or their un-added split-K sums (PartialSums); q and
    k are rotated by ``cos_sin`` [rows, hd/2, 2] (None: not rotated), k and v stored at ``slots``
    (None: nothing stored), and every row attends over its whole context.  One launch; with
    ``max_context`` (a bound of every row's context length) beyond 1,024 and few rows, contexts are
    cut into parts that a second small launch merges, which needs ``scratch``
    (attention_decode_fused_scratch floats; allocated here when not given)."""
    partial = isinstance(projection, PartialSums)
    rows_t = projection.out if partial else projection
    T = rows_t.shape[0] if rows is None else rows
    _dev(rows_t, out, kcache, vcache, tables, row_seq, ctx_lens, cos_sin, slots)
    _rows2d(out, "out")
    width = (nh + 2 * nkv) * hd
    _need(out.dtype == kcache.dtype == vcache.dtype == torch.bfloat16, "attention_decode_fused is bfloat16 only")
    _check_caches(kcache, vcache, nkv, hd, packed_offsets=True)
    if partial:
        _need(projection.cols == width and projection.rows == T, "the partial sums are not [splits, rows, (nh + 2 nkv) * hd]")
    else:
        _rows2d(rows_t, "qkv")
        _need(rows_t.dtype == torch.bfloat16 and rows_t.shape[1] >= width and rows_t.shape[0] >= T, "qkv must be bfloat16 [rows, (nh + 2 nkv) * hd]")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.numel() >= T * hd, "cos_sin must be float32 [rows, hd/2, 2]")
    if slots is not None:
        _i32(slots, "slots", T)
    _i32(row_seq, "row_seq", T)
    _i32(ctx_lens, "ctx_lens", T)
    _i32(tables, "tables")
    _need(out.shape[0] >= T and out.shape[1] >= nh * hd, "out must be [rows, nh * hd]")
    need = attention_decode_fused_scratch(T, nh, nkv, hd, int(max_context))
    if need and scratch is None:
        _need(_recording is None, "attention_decode_fused: a recorded step must bring its scratch (an allocation here would not outlive the step)")
        scratch = torch.empty(need, dtype=torch.float32, device=out.device)
    if scratch is not None:
        _dev(scratch)
        _need(scratch.dtype == torch.float32 and scratch.is_contiguous(), "scratch must be contiguous float32")
    _call("kvcm_attention_decode_fused", 
        _ptr(projection.data) if partial else 0, projection.splits if partial else 0,
        0 if partial else _ptr(rows_t), 0 if partial else rows_t.stride(0), _ptr(cos_sin), _ptr(slots), _ptr(kcache),
        _ptr(vcache), _ptr(tables), table_stride, _ptr(row_seq), _ptr(ctx_lens), T, nh, nkv, hd, kcache.shape[2],
        float(scale), _ptr(out), out.stride(0), int(max_context), _ptr(scratch),
        scratch.numel() if scratch is not None else 0, _stream())


def attention_prefill_supported(nh, nkv, hd, dtype, block_size=16):
    return dtype == torch.bfloat16 and bool(lib().kvcm_attention_prefill_supported(nh, nkv, hd, block_size))


def attention_prefill_scratch(rows, nh, hd, max_context, max_run, num_seqs):
    """Floats of scratch ``attention_prefill`` needs for a launch of these sizes (0 while contexts
    fit one segment of keys)."""
    return int(lib().kvcm_attention_prefill_scratch(rows, nh, hd, max_context, max_run, num_seqs))


def attention_prefill_segment(rows, nh, hd, max_context, max_run, num_seqs):
    """Keys per segment that a launch of these sizes cuts contexts into."""
    return int(lib().kvcm_attention_prefill_segment(rows, nh, hd, max_context, max_run, num_seqs))


def attention_prefill_tile_rows(rows, nh, hd, max_context, max_run, num_seqs):
    """Query rows per workgroup of a launch of these sizes (128; 64 for small launches at head_dim 64)."""
    return int(lib().kvcm_attention_prefill_tile_rows(rows, nh, hd, max_context, max_run, num_seqs))


def attention_prefill(q, out, kcache, vcache, tables, table_stride, run_start, seq_start, num_seqs, max_run, nh, nkv, hd,
                      scale, rows=None, max_context=None, scratch=None, cos_sin=None):
    """Causal attention for runs of consecutive positions (bfloat16): sequence s owns rows
    run_start[s] .. run_start[s+1]-1, the first of them at position seq_start[s]; every row sees the
    sequence's cached tokens up to its own position.  The same result as ``attention``.
    ``cos_sin`` (float32 [rows, hd/2, 2]): q is not rotated yet; the kernel rotates it with this table
    as it reads it (the keys in the cache are rotated already).
    ``rows``: rows in all; ``max_context``: a bound of every row's context length (default: what the
    block tables can hold); contexts beyond one segment of keys need ``scratch`` (float32,
    attention_prefill_scratch elements; allocated here when not given)."""
    _dev(q, out, kcache, vcache, tables, run_start, seq_start, scratch)
    T = q.shape[0] if rows is None else rows
    if max_context is None:
        max_context = table_stride * kcache.shape[2]
    need = attention_prefill_scratch(T, nh, hd, max_context, max_run, num_seqs)
    if need and scratch is None:
        _need(_recording is None, "attention_prefill: a recorded step must bring its scratch (an allocation here would not outlive the step)")
        scratch = torch.empty(need, dtype=torch.float32, device=q.device)
    if scratch is not None:
        _need(scratch.dtype == torch.float32 and scratch.is_contiguous(), "scratch must be contiguous float32")
    _rows2d(q, "q")
    _rows2d(out, "out")
    _need(q.dtype == out.dtype == kcache.dtype == vcache.dtype == torch.bfloat16, "attention_prefill is bfloat16 only")
    _check_caches(kcache, vcache, nkv, hd)
    _i32(run_start, "run_start", num_seqs + 1)
    _i32(seq_start, "seq_start", num_seqs)
    _i32(tables, "tables", num_seqs * table_stride)
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.numel() >= T * hd
              and cos_sin.is_cuda, "cos_sin must be float32 [rows, head_dim/2, 2]")
    _call("kvcm_attention_prefill", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(kcache), _ptr(vcache),
                                        _ptr(tables), table_stride, _ptr(run_start), _ptr(seq_start), num_seqs, max_run,
                                        T, int(max_context), nh, nkv, hd, kcache.shape[2], float(scale), _ptr(scratch),
                                        scratch.numel() if scratch is not None else 0, _ptr(cos_sin), _stream())


# ------------------------------------------------------------------------- probes of the machine
def probe_empty(grid=1, block=64):
    _check(lib().kvcm_probe_empty(int(grid), int(block), _stream()))


def probe_copy(src, dst, grid=2048):
    """dst = src + 1 over 16-byte pieces; moves 2 * src.nbytes."""
    _dev(src, dst)
    n = src.numel() * src.element_size()
    _need(src.is_contiguous() and dst.is_contiguous() and dst.numel() * dst.element_size() >= n and n % 16 == 0, "probe_copy needs contiguous buffers of whole 16-byte pieces")
    _check(lib().kvcm_probe_copy(_ptr(src), _ptr(dst), n, int(grid), _stream()))


def probe_read(src, sink, grid=2048, nbytes=None):
    _dev(src, sink)
    n = src.numel() * src.element_size() if nbytes is None else int(nbytes)
    _need(src.is_contiguous() and n % 16 == 0 and n <= src.numel() * src.element_size() and sink.numel() * sink.element_size() >= 1024, "probe_read needs whole 16-byte pieces and a sink of 1 KiB")
    _check(lib().kvcm_probe_read(_ptr(src), n, _ptr(sink), int(grid), _stream()))


def probe_stream(src, sink, grid, waves=4, inflight=8):
    """``src`` read once by ``grid`` workgroups of ``waves`` waves, a contiguous share each."""
    _dev(src, sink)
    n = src.numel() * src.element_size()
    _need(src.is_contiguous() and n % 16 == 0 and sink.numel() * sink.element_size() >= 1024, "probe_stream needs whole 16-byte pieces and a sink of 1 KiB")
    _check(lib().kvcm_probe_stream(_ptr(src), n, _ptr(sink), int(grid), int(waves), int(inflight), _stream()))


def probe_mfma(iters, sink, grid=2048):
    """-> flops of the launch: grid workgroups x 4 waves x iters x 4 instructions x 32768."""
    _dev(sink)
    _need(sink.numel() * sink.element_size() >= 1024, "probe_mfma needs a sink of 1 KiB")
    _check(lib().kvcm_probe_mfma(int(iters), _ptr(sink), int(grid), _stream()))
    return int(grid) * 4 * int(iters) * 4 * 32768


def probe_barrier(data, counter, flags, workgroups, rounds, spin_cap=1 << 16, fences=False, awaited=None):
    """``rounds`` barriers across ``workgroups`` workgroups of one launch (counter: zero before the launch).
    ``awaited``: the arrivals a barrier waits for, the launch's workgroups unless a test of the bounded wait
    names one more (who never comes: every workgroup then polls ``spin_cap`` times, raises flags[0] and leaves)."""
    _dev(data, counter, flags)
    _need(data.numel() >= 2 * workgroups * 256 and data.dtype == torch.float32 and counter.dtype == flags.dtype == torch.int32
          and flags.numel() >= 2, "probe_barrier: data float32 [2, workgroups, 256], counter int32 [1], flags int32 [2]")
    _check(lib().kvcm_probe_barrier(_ptr(data), _ptr(counter), _ptr(flags), int(workgroups), int(rounds), int(spin_cap), int(fences),
                                    int(workgroups if awaited is None else awaited), _stream()))


def probe_sums(partials, counters, out, splits, tiles, last_arriver, flags):
    _dev(partials, counters, out, flags)
    _need(partials.numel() >= splits * tiles * 1024 and out.numel() >= tiles * 1024 and counters.numel() >= tiles
          and partials.dtype == out.dtype == torch.float32 and counters.dtype == flags.dtype == torch.int32 and flags.numel() >= 2,
          "probe_sums: partials float32 [tiles, splits, 1024], out float32 [tiles, 1024], counters int32 [tiles], flags int32 [2]")
    _check(lib().kvcm_probe_sums(_ptr(partials), _ptr(counters), _ptr(out), int(splits), int(tiles), int(last_arriver), _ptr(flags), _stream()))


def probe_phases(weights, phase_bytes, layers, persistent, workgroups=256, counters=None, act=None, flags=None, sink=None, spin_cap=1 << 18):
    """A step of ``layers`` x len(phase_bytes) dependent phases over ``weights`` (four layers' bytes): as one
    launch (``persistent``) or as one launch per phase."""
    _dev(weights, counters, act, flags, sink)
    layer = sum(phase_bytes)
    _need(weights.numel() * weights.element_size() >= 4 * layer, "probe_phases: weights must hold four layers' bytes")
    if persistent:
        _need(counters is not None and counters.numel() >= layers * len(phase_bytes) * 17 and act is not None and act.numel() >= 8192
              and flags is not None and flags.numel() >= 2, "probe_phases: counters int32 [layers * phases * 17], act float32 [8192], flags int32 [2]")
    arr = (C.c_longlong * len(phase_bytes))(*[int(b) for b in phase_bytes])
    _check(lib().kvcm_probe_phases(_ptr(weights), arr, len(phase_bytes), int(layers), int(bool(persistent)), int(workgroups), _ptr(counters),
                                   _ptr(act), _ptr(flags), _ptr(sink), int(spin_cap), _stream()))


def fill_normal(out, key, mean=0.0, std=1.0):
    """out[i] = mean + std * n(key, i) over the flattened tensor: the counter-based normal values of
    weights/random_init.py, made on the device (float32 or bfloat16)."""
    _dev(out)
    _need(out.is_contiguous() and out.dtype in _DT, "fill_normal needs a contiguous float32 or bfloat16 tensor")
    _check(lib().kvcm_fill_normal(_ptr(out), _DT[out.dtype], out.numel(), int(key) & _MASK64, float(mean), float(std), _stream()))
    return out


def fill_index(out, key, modulus):
    _dev(out)
    _need(out.is_contiguous() and out.dtype == torch.int32 and modulus > 0, "fill_index needs a contiguous int32 tensor")
    _check(lib().kvcm_fill_index(_ptr(out), out.numel(), int(key) & _MASK64, int(modulus), _stream()))
    return out


def sample(logits, out, temperature=None, seeds=None, request_ids=None, token_index=None):
    """out[r] = argmax of row r, or a Gumbel-max draw where temperature[r] > 0."""
    _dev(logits, out, temperature, seeds, request_ids, token_index)
    _rows2d(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    _i32(out, "out", R)
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and temperature.numel() >= R, "temperature must be float32 [R]")
        _need(seeds is not None and seeds.dtype in (torch.int64, torch.uint64) and seeds.numel() >= R, "seeds must be 64-bit [R]")
        _need(request_ids is not None and request_ids.dtype == torch.int64 and request_ids.numel() >= R, "request ids must be int64 [R]")
        _i32(token_index, "token_index", R)
    _call("kvcm_sample", _ptr(logits), logits.stride(0), _ptr(temperature), _ptr(seeds), _ptr(request_ids),
                             _ptr(token_index), _ptr(out), R, V, _stream())


# ------------------------------------------------------------- parts of other sequence models
GATE_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2}


def _f32(t, name, n=None):
    if t is None:
        return
    _need(t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda, f"{name} must be a contiguous float32 tensor on the GPU")
    if n is not None:
        _need(t.numel() >= n, f"{name} holds {t.numel()} values, {n} are needed")


def _f32rows(t, name, cols):
    _need(t.dtype == torch.float32 and t.is_cuda and t.dim() == 2 and t.stride(1) == 1 and t.shape[1] >= cols,
          f"{name} must be float32 rows of at least {cols} columns")


def embed_scaled(ids, table, out, factor):
    """out[t, :] = float(table[ids[t], :]) * factor."""
    _dev(ids, table, out)
    T, H = out.shape
    _i32(ids, "ids", T)
    _need(table.dim() == 2 and table.shape[1] == H and table.is_contiguous(), "embedding table must be [V, H]")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "residual stream must be contiguous float32")
    _call("kvcm_embed_scaled", _ptr(ids), _ptr(table), _DT[table.dtype], _ptr(out), T, H, table.shape[0], float(factor), _stream())


def gated_act(gate_up, out, activation):
    """out[T, I] = act(gate) * up for 32-bit rows [gate (I) | up (I)]; act: "silu", "relu" or "gelu_tanh"."""
    T, I = out.shape
    _f32rows(gate_up, "gate_up", 2 * I)
    _rows2d(out, "out")
    _need(gate_up.shape[0] >= T and out.is_cuda, "gated_act: the rows do not agree")
    _need(activation in GATE_ACTIVATIONS, f"unknown activation {activation!r} ({sorted(GATE_ACTIVATIONS)})")
    _call("kvcm_gated_act", _ptr(gate_up), gate_up.stride(0), _ptr(out), _DT[out.dtype], out.stride(0), T, I,
          GATE_ACTIVATIONS[activation], _stream())


class NormedBranches:
    """A sublayer's output that is still to be normed and added to the residual stream:
    x += n(m) * w_post with m = a, or m = combine * (n(a) * wa + n(b) * wb) for two branches side by side
    (n: division by the root mean square).  ``rmsnorm_chain`` consumes it; ``materialize`` is not offered:
    the addition belongs to the stream's next reader."""

    def __init__(self, a, w_post, b=None, wa=None, wb=None, combine=1.0):
        self.a, self.b, self.wa, self.wb, self.combine, self.w_post = a, b, wa, wb, float(combine), w_post


def rmsnorm_chain(x, eps, pending=None, weight=None, out=None, rows=None, plain=False):
    """x += the pending output (NormedBranches), normed; then out[r] = n(x[src]) * weight, src = rows[r] or r
    (``plain``: out[r] = x[src], for a reader of the stream as it is).
    All arithmetic is 32-bit; ``out`` is rounded once to its dtype.  With ``rows`` the stream is not written."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.is_cuda and x.dim() == 2, "x must be contiguous float32 [T, H]")
    T, H = x.shape
    a = b = wa = wb = wp = None
    combine, a_splits, b_splits = 1.0, 1, 1
    if pending is not None:
        a, b, wa, wb, wp, combine = pending.a, pending.b, pending.wa, pending.wb, pending.w_post, pending.combine
        # a branch may be the un-added slices of a split product (PartialSums [splits][T][H]): they are added here
        if isinstance(a, PartialSums):
            _need(a.rows == T and a.cols == H, "a branch's partial sums must match x")
            a, a_splits = a.data, a.splits
        elif a is not None:
            _need(a.dtype == torch.float32 and a.is_contiguous() and a.shape == x.shape, "branch a must match x")
        if isinstance(b, PartialSums):
            _need(b.rows == T and b.cols == H, "a branch's partial sums must match x")
            b, b_splits = b.data, b.splits
        elif b is not None:
            _need(b.dtype == torch.float32 and b.is_contiguous() and b.shape == x.shape, "branch b must match x")
        for t in (wa, wb, wp):
            _f32(t, "a norm weight", H)
    R = T
    if out is not None:
        _need(out.is_cuda and out.is_contiguous() and out.dim() == 2 and out.shape[1] == H, "out must be contiguous [R, H]")
        if plain:
            weight = None
        else:
            _need(weight is not None, "rmsnorm_chain: a normed output needs its weight")
            _f32(weight, "the norm weight", H)
        R = out.shape[0]
        if rows is not None:
            _i32(rows, "rows", R)
        else:
            _need(R <= T, "x has fewer rows than the output")
    else:
        _need(pending is not None and rows is None, "rmsnorm_chain: nothing to do")
    _call("kvcm_rmsnorm_chain", _ptr(x), _ptr(a), a_splits, _ptr(b), b_splits, T * H, _ptr(wa), _ptr(wb), combine, _ptr(wp), _ptr(rows), _ptr(weight),
          _ptr(out), _DT[out.dtype] if out is not None else 0, R, H, float(eps), _stream())
    return out


def head_norm_gate(o, gate, weight, out, heads, d, eps):
    """out[r, h, :] = n(o[r, h, :]) * weight[h, :] * sigmoid(gate[r, h, :])."""
    T = out.shape[0]
    _f32rows(o, "o", heads * d)
    _f32rows(gate, "gate", heads * d)
    _f32(weight, "weight", heads * d)
    _rows2d(out, "out")
    _need(o.shape[0] >= T and gate.shape[0] >= T and out.shape[1] >= heads * d and out.is_cuda, "head_norm_gate: shapes do not agree")
    _call("kvcm_head_norm_gate", _ptr(o), o.stride(0), _ptr(gate), gate.stride(0), _ptr(weight), _ptr(out), _DT[out.dtype],
          out.stride(0), T, heads, d, float(eps), _stream())
    return out


def short_conv(x, weight, out, step, state, bias_in=None, bias_out=None, activation=None, rows=None, update_state=False):
    """Causal convolution per channel over the step's packed runs.  x: 32-bit rows [T, >= C]; weight [C, taps];
    state [slots, taps-1, C] (the sequences' last inputs, read here); out [T, >= C].  ``step`` brings row_seq,
    positions, ctx_lens, run_start, seq_start, state_slots.  ``update_state``: for steps in which every sequence runs one
    row only; the rows then leave the new state themselves and ``short_conv_state`` is not called."""
    C, taps = weight.shape
    T = out.shape[0] if rows is None else rows
    _f32rows(x, "x", C)
    _f32(weight, "weight")
    _f32(bias_in, "bias_in", C)
    _f32(bias_out, "bias_out", C)
    _rows2d(out, "out")
    _need(out.shape[1] >= C and out.is_cuda and x.shape[0] >= T, "short_conv: shapes do not agree")
    if taps > 1:
        _need(state is not None and state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 3
              and tuple(state.shape[1:]) == (taps - 1, C), "state must be float32 [slots, taps-1, C]")
    _need(activation in (None, "silu"), "short_conv: activation is None or 'silu'")
    for name in ("row_seq", "positions", "ctx_lens"):
        _i32(getattr(step, name), name, T)
    _call("kvcm_short_conv", _ptr(x), x.stride(0), _ptr(bias_in), _ptr(weight), _ptr(bias_out), _ptr(state), _ptr(out),
          _DT[out.dtype], out.stride(0), _ptr(step.row_seq), _ptr(step.positions), _ptr(step.ctx_lens), _ptr(step.run_start),
          _ptr(step.seq_start), _ptr(step.state_slots), T, C, taps, 1 if activation == "silu" else 0,
          1 if (update_state and taps > 1) else 0, _stream())
    return out


def short_conv_state(x, state, step, taps, bias_in=None):
    """Leaves every sequence's last taps-1 inputs (after this step's rows) in its slot of ``state``."""
    if taps <= 1:
        return
    C = state.shape[2]
    _f32rows(x, "x", C)
    _f32(bias_in, "bias_in", C)
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.is_cuda and tuple(state.shape[1:]) == (taps - 1, C),
          "state must be float32 [slots, taps-1, C]")
    _call("kvcm_short_conv_state", _ptr(x), x.stride(0), _ptr(bias_in), _ptr(state), _ptr(step.run_start), _ptr(step.seq_start),
          _ptr(step.seq_end), _ptr(step.state_slots), step.seqs, C, taps, _stream())


def rotary_pairs_table(positions, out, dims, base, rows=None):
    """out[t, i] = (cos, sin) of positions[t] * base^(-2i/dims), float32 [rows, dims/2, 2]."""
    T = out.shape[0] if rows is None else rows
    _i32(positions, "positions", T)
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.is_cuda and out.numel() >= T * dims,
          "the table must be float32 [rows, dims/2, 2]")
    _call("kvcm_rotary_pairs_table", _ptr(positions), _ptr(out), T, dims, float(base), _stream())
    return out


def rotate_store(qkv, q_out, nh, nkv, d, dv, cos_sin=None, rot=0, slots=None, kcache=None, vcache=None, rows=None, halves=False,
                 kv=None):
    """qkv: 32-bit rows [q (nh*d) | k (nkv*d) | v (nkv*dv)]; or q alone there and ``kv``: 32-bit rows [k | v] of their
    own; without ``slots`` only q is read.  The first ``rot`` entries of every q and k head are
    turned with the table ``cos_sin``, by interleaved pairs (2i, 2i+1) or, with ``halves``, by pairs (i, i + rot/2);
    q goes to q_out [T, nh*d], k and v to their page slots (keys [pages, nkv, B, d], values [pages, nkv, dv, B])."""
    T = q_out.shape[0] if rows is None else rows
    if kv is not None:
        _f32rows(qkv, "q", nh * d)
        _f32rows(kv, "kv", nkv * (d + dv))
        _need(kv.shape[0] >= T, "rotate_store: kv has fewer rows than the step")
    else:
        _f32rows(qkv, "qkv", (nh + nkv) * d + nkv * dv if slots is not None else nh * d)
    _rows2d(q_out, "q_out")
    _need(q_out.shape[1] >= nh * d and q_out.is_cuda and qkv.shape[0] >= T, "rotate_store: shapes do not agree")
    B = 1
    if slots is not None:
        _i32(slots, "slots", T)
        _need(kcache is not None and kcache.dtype == q_out.dtype and kcache.is_contiguous() and kcache.dim() == 4
              and kcache.shape[1] == nkv and kcache.shape[3] == d, "key cache must be [pages, nkv, block_size, d]")
        B = kcache.shape[2]
        _need(vcache is not None and vcache.dtype == q_out.dtype and vcache.is_contiguous()
              and tuple(vcache.shape) == (kcache.shape[0], nkv, dv, B), "value cache must be [pages, nkv, dv, block_size]")
    if rot:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.numel() >= T * rot,
              "cos_sin must be float32 [rows, rot/2, 2]")
    _call("kvcm_rotate_store", _ptr(qkv), qkv.stride(0), _ptr(kv), kv.stride(0) if kv is not None else 0, _ptr(cos_sin), rot, 1 if halves else 0, _ptr(slots), _ptr(q_out), _DT[q_out.dtype],
          q_out.stride(0), _ptr(kcache), _ptr(vcache), T, nh, nkv, d, dv, B, _stream())


def norm_rotate_store(qkv, q_out, nh, nkv, d, dv, eps, q_weight=None, k_weight=None, v_other=None, mix=0.0, v_keep=None,
                      cos_sin=None, rot=0, slots=None, kcache=None, vcache=None, rows=None, halves=False):
    """``rotate_store`` after what some attentions do to the projection first: q and k are each divided by the root mean
    square over their whole stretch of the row (all heads at once; eps inside the root) and multiplied by ``q_weight``
    [nh*d] / ``k_weight`` [nkv*d] (None: that stretch passes); v <- (1 - mix) v + mix * v_other where ``v_other``
    (float32 rows of nkv*dv: another layer's values of the same rows) is given; ``v_keep`` (float32 rows) receives the
    values as the projection made them.  The blended v goes to the pages."""
    T = q_out.shape[0] if rows is None else rows
    _f32rows(qkv, "qkv", (nh + nkv) * d + nkv * dv)
    _rows2d(q_out, "q_out")
    _need(q_out.shape[1] >= nh * d and q_out.is_cuda and qkv.shape[0] >= T, "norm_rotate_store: shapes do not agree")
    _f32(q_weight, "q_weight", nh * d)
    _f32(k_weight, "k_weight", nkv * d)
    for t, name in ((v_other, "v_other"), (v_keep, "v_keep")):
        if t is not None:
            _f32rows(t, name, nkv * dv)
            _need(t.shape[0] >= T, f"{name} has fewer rows than the step")
    B = 1
    if slots is not None:
        _i32(slots, "slots", T)
        _need(kcache is not None and kcache.dtype == q_out.dtype and kcache.is_contiguous() and kcache.dim() == 4
              and kcache.shape[1] == nkv and kcache.shape[3] == d, "key cache must be [pages, nkv, block_size, d]")
        B = kcache.shape[2]
        _need(vcache is not None and vcache.dtype == q_out.dtype and vcache.is_contiguous()
              and tuple(vcache.shape) == (kcache.shape[0], nkv, dv, B), "value cache must be [pages, nkv, dv, block_size]")
    if rot:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.numel() >= T * rot,
              "cos_sin must be float32 [rows, rot/2, 2]")
    _call("kvcm_norm_rotate_store", _ptr(qkv), qkv.stride(0), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(v_other),
          v_other.stride(0) if v_other is not None else 0, float(mix), _ptr(v_keep), v_keep.stride(0) if v_keep is not None else 0,
          _ptr(cos_sin), rot, 1 if halves else 0, _ptr(slots), _ptr(q_out), _DT[q_out.dtype], q_out.stride(0), _ptr(kcache),
          _ptr(vcache), T, nh, nkv, d, dv, B, _stream())


def _check_pool(kcache, vcache, pk, pv, nkv, d, dv, P):
    B = kcache.shape[2]
    _need(kcache.dim() == 4 and kcache.is_contiguous() and kcache.shape[1] == nkv and kcache.shape[3] == d,
          "key cache must be [pages, nkv, block_size, d]")
    _need(vcache.is_contiguous() and tuple(vcache.shape) == (kcache.shape[0], nkv, dv, B) and vcache.dtype == kcache.dtype,
          "value cache must be [pages, nkv, dv, block_size]")
    E = 0
    if P > 0:
        E = (B + P - 1) // P
        _need(pk is not None and pk.dtype == torch.float32 and pk.is_contiguous() and tuple(pk.shape) == (kcache.shape[0], nkv, E, d),
              "pooled keys must be float32 [pages, nkv, ceil(block_size / pool), d]")
        _need(pv is not None and pv.dtype == torch.float32 and pv.is_contiguous() and tuple(pv.shape) == (kcache.shape[0], nkv, E, dv),
              "pooled values must be float32 [pages, nkv, ceil(block_size / pool), dv]")
    return B, E


def pool_update(kcache, vcache, pk, pv, tables, table_stride, row_seq, positions, slots, nkv, d, dv, P, rows):
    """Every row whose position ends a block of P tokens leaves that block's mean key and mean value with its page."""
    if P <= 0:
        return
    _dev(kcache, vcache, pk, pv, tables, row_seq, positions, slots)
    B, E = _check_pool(kcache, vcache, pk, pv, nkv, d, dv, P)
    for t, n in ((row_seq, "row_seq"), (positions, "positions"), (slots, "slots")):
        _i32(t, n, rows)
    _i32(tables, "tables")
    _call("kvcm_pool_update", _ptr(kcache), _ptr(vcache), _DT[kcache.dtype], _ptr(pk), _ptr(pv), _ptr(tables), table_stride,
          _ptr(row_seq), _ptr(positions), _ptr(slots), rows, nkv, d, dv, B, P, E, _stream())


def attention_window_pool(q, out, kcache, vcache, pk, pv, tables, table_stride, row_seq, ctx_lens, nh, nkv, d, dv, scale,
                          window, P, head_scale=None, rows=None, keep_first=0, softcap=0.0, dist_slope=None, gate=None):
    """out[r, h] = softmax over the last ``window`` tokens, the sequence's first ``keep_first`` tokens and the pooled
    blocks of P tokens before the window (window 0: every token, no blocks) of (q . k) * scale * head_scale[h], times the
    values.  ``softcap`` c > 0: the scores are capped first, c tanh(score / c).  ``dist_slope`` (float32 [nh]): a bias that
    grows with the distance is taken off the scores, slope[h] * (query position - key position).  ``gate`` (float32 rows of
    >= nh*dv): the output is multiplied element by element with sigmoid(gate) before it is stored."""
    _dev(q, out, kcache, vcache, tables, row_seq, ctx_lens)
    _rows2d(q, "q")
    _rows2d(out, "out")
    T = q.shape[0] if rows is None else rows
    _need(q.dtype == out.dtype == kcache.dtype, "attention operands must share one dtype")
    _need(q.shape[1] >= nh * d and out.shape[1] >= nh * dv, "attention rows are too short for the head layout")
    B, E = _check_pool(kcache, vcache, pk, pv, nkv, d, dv, P)
    _f32(head_scale, "head_scale", nh)
    _f32(dist_slope, "dist_slope", nh)
    if gate is not None:
        _f32rows(gate, "gate", nh * dv)
        _need(gate.shape[0] >= T, "attention_window_pool: the gate has fewer rows than the step")
    _i32(row_seq, "row_seq", T)
    _i32(ctx_lens, "ctx_lens", T)
    _i32(tables, "tables")
    _call("kvcm_attention_window_pool", _ptr(q), _DT[q.dtype], q.stride(0), _ptr(out), out.stride(0), _ptr(kcache), _ptr(vcache),
          _ptr(pk), _ptr(pv), _ptr(tables), table_stride, _ptr(row_seq), _ptr(ctx_lens), _ptr(head_scale), _ptr(dist_slope), _ptr(gate),
          gate.stride(0) if gate is not None else 0, T, nh, nkv, d, dv,
          B, float(scale), int(window), int(P), E, int(keep_first), float(softcap or 0.0), _stream())


def attention_window_pool_tiles_supported(d, dv, dtype, block_size):
    """Does the matrix-core kernel for runs of consecutive positions take this head shape?"""
    return dtype == torch.bfloat16 and bool(lib().kvcm_attention_window_pool_tiles_supported(d, dv, block_size))


def attention_window_pool_tiles(q, out, kcache, vcache, pk, pv, tables, table_stride, run_start, seq_start, num_seqs, max_run,
                                nh, nkv, d, dv, scale, window, P, head_scale=None, keep_first=0, softcap=0.0, dist_slope=None, gate=None):
    """``attention_window_pool`` for steps whose sequences run several consecutive positions: 64 rows of a run and one
    head per workgroup on the matrix cores (bfloat16 only).  Every row of every run is computed, single rows too."""
    _dev(q, out, kcache, vcache, tables, run_start, seq_start)
    _rows2d(q, "q")
    _rows2d(out, "out")
    _need(q.dtype == out.dtype == kcache.dtype == torch.bfloat16, "the tiled attention takes bfloat16 operands")
    _need(q.shape[1] >= nh * d and out.shape[1] >= nh * dv, "attention rows are too short for the head layout")
    B, E = _check_pool(kcache, vcache, pk, pv, nkv, d, dv, P)
    _f32(head_scale, "head_scale", nh)
    _f32(dist_slope, "dist_slope", nh)
    if gate is not None:
        _f32rows(gate, "gate", nh * dv)
        _need(gate.shape[0] >= out.shape[0], "attention_window_pool_tiles: the gate has fewer rows than the output")
    _i32(run_start, "run_start", num_seqs + 1)
    _i32(seq_start, "seq_start", num_seqs)
    _i32(tables, "tables")
    _call("kvcm_attention_window_pool_tiles", _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(kcache), _ptr(vcache), _ptr(pk),
          _ptr(pv), _ptr(tables), table_stride, _ptr(run_start), _ptr(seq_start), _ptr(head_scale), _ptr(dist_slope), _ptr(gate),
          gate.stride(0) if gate is not None else 0, num_seqs, max_run, nh, nkv,
          d, dv, B, float(scale), int(window), int(P), E, int(keep_first), float(softcap or 0.0), _stream())


SCAN_PIECE = 128      # rows of a piece when long runs are walked in pieces


def selective_scan_carry_floats(rows, seqs, C, N, piece=SCAN_PIECE):
    """32-bit values of scratch that ``selective_scan(..., pieces=True)`` needs for a step of this shape."""
    return (rows // piece + seqs + 1) * C * (N + 1)


def selective_scan(x, dt_lin, dt_bias, bc, off_b, off_c, a_log, dskip, z, out, state, step, prepare=False, carry=None):
    """The selective scan of the step's runs (csrc/hip/selective_scan.hip).  x, out [T, C] in the compute dtype;
    dt_lin [T, C], bc rows with B at off_b and C at off_c, z rows: 32-bit; state [slots, C, N].  ``prepare``: the step
    sizes and gates of all rows are made first, in place in dt_lin and z, by a launch of their own (pays for long runs).
    ``carry`` (float32 scratch of ``selective_scan_carry_floats``; needs ``prepare``): runs are walked in pieces of
    SCAN_PIECE rows, all pieces at once: each from zero, then the states that enter the pieces (a short walk over the
    pieces' ends), then each again from its entering state.  The sums are the token-by-token ones in another order."""
    C, N = a_log.shape
    _rows2d(x, "x")
    _rows2d(out, "out")
    _need(x.dtype == out.dtype and x.is_cuda and x.shape[1] >= C and out.shape[1] >= C, "selective_scan: x and out do not agree")
    _f32rows(dt_lin, "dt_lin", C)
    _f32rows(bc, "bc", max(off_b, off_c) + N)
    _f32rows(z, "z", C)
    _f32(dt_bias, "dt_bias", C)
    _f32(a_log, "a_log")
    _f32(dskip, "dskip", C)
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.is_cuda and tuple(state.shape[1:]) == (C, N),
          "state must be float32 [slots, C, N]")
    if carry is not None:
        _need(prepare and carry.dtype == torch.float32 and carry.is_contiguous() and carry.is_cuda
              and carry.numel() >= selective_scan_carry_floats(out.shape[0], step.seqs, C, N), "the scratch for the pieces is too small")
    if prepare:
        _call("kvcm_scan_prepare", _ptr(dt_lin), dt_lin.stride(0), _ptr(dt_bias), _ptr(z), z.stride(0), out.shape[0], C, _stream())
    _call("kvcm_selective_scan", _ptr(x), _DT[x.dtype], x.stride(0), _ptr(dt_lin), dt_lin.stride(0), _ptr(dt_bias), _ptr(bc),
          bc.stride(0), off_b, off_c, _ptr(a_log), _ptr(dskip), _ptr(z), z.stride(0), _ptr(out), out.stride(0), _ptr(state),
          _ptr(step.run_start), _ptr(step.seq_start), _ptr(step.state_slots), step.seqs, C, N, 1 if prepare else 0,
          SCAN_PIECE if carry is not None else 0, step.max_run, _ptr(carry), carry.numel() if carry is not None else 0,
          out.shape[0], _stream())
    return out


def delta_prepare(k, a_lin, a_bias, low, w2t, w0, w_out, au_out, u_out, heads, d, rows):
    """(decay, removal rate times unit key, unit key) of every row and head from the projections; ``low`` is the
    first step of the decay's projection [T, rank], ``w2t`` [rank, heads*d] its second step's matrix, transposed."""
    D = heads * d
    for t, n in ((k, "k"), (a_lin, "a_lin")):
        _f32rows(t, n, D)
    rank = w2t.shape[0]
    _f32rows(low, "low", rank)
    _need(w2t.dtype == torch.float32 and w2t.is_contiguous() and w2t.is_cuda and w2t.shape[1] == D, "w2t must be contiguous float32 [rank, heads*d]")
    for t, n in ((a_bias, "a_bias"), (w0, "w0")):
        _f32(t, n, D)
    for t, n in ((w_out, "w_out"), (au_out, "au_out"), (u_out, "u_out")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda and t.shape[0] >= rows and t.shape[1] == D,
              f"{n} must be contiguous float32 [T, heads*d]")
    _call("kvcm_delta_prepare", _ptr(k), k.stride(0), _ptr(a_lin), a_lin.stride(0), _ptr(a_bias), _ptr(low), low.stride(0),
          _ptr(w2t), rank, _ptr(w0), _ptr(w_out), _ptr(au_out), _ptr(u_out), rows, heads, d, _stream())


def delta_scan(r, k, v, w, au, u, o, state, step, heads, dk, dv):
    """The delta-rule recurrence over the step's runs (csrc/hip/delta_rule.hip); state [slots, heads, dk, dv]."""
    for t, n, c in ((r, "r", heads * dk), (k, "k", heads * dk), (v, "v", heads * dv), (o, "o", heads * dv)):
        _f32rows(t, n, c)
    for t, n in ((w, "w"), (au, "au"), (u, "u")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda and t.shape[1] == heads * dk, f"{n} must be contiguous float32")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.is_cuda and tuple(state.shape[1:]) == (heads, dk, dv),
          "state must be float32 [slots, heads, dk, dv]")
    _call("kvcm_delta_scan", _ptr(r), r.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(w), _ptr(au), _ptr(u),
          _ptr(o), o.stride(0), _ptr(state), _ptr(step.run_start), _ptr(step.seq_start), _ptr(step.state_slots), step.seqs,
          heads, dk, dv, _stream())
    return o


# ------------------------------------------- a stream whose layers run mixer and feed-forward side by side
def rotary_freq_table(positions, freqs, out, dims, factor=1.0, rows=None):
    """out[t, i] = factor * (cos, sin) of positions[t] * freqs[i], float32 [rows, dims/2, 2]; freqs: float64 [dims/2] on
    the GPU (frequencies that are no plain power law: rescaled pair by pair for longer contexts)."""
    T = out.shape[0] if rows is None else rows
    _i32(positions, "positions", T)
    _need(freqs.dtype == torch.float64 and freqs.is_contiguous() and freqs.is_cuda and freqs.numel() == dims // 2,
          "freqs must be float64 [dims/2] on the GPU")
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.is_cuda and out.numel() >= T * dims,
          "the table must be float32 [rows, dims/2, 2]")
    _call("kvcm_rotary_freq_table", _ptr(positions), _ptr(freqs), _ptr(out), T, dims, float(factor), _stream())
    return out


class DytNorm:
    """One norm tanh(alpha x) * weight + bias as ``dyt_norm`` takes it: (weight, bias: float32 [H]; alpha: a number)."""

    def __init__(self, weight, bias, alpha):
        self.weight, self.bias, self.alpha = weight, bias, float(alpha)


def dyt_norm(x, first=None, out1=None, second=None, out2=None, add_a=None, add_b=None, rows=None, replace=False):
    """x += add_a + add_b (``replace``: x = add_a + add_b), written back unless ``rows`` gathers; then
    out1 = first(x), out2 = second(x), each tanh(alpha x) * weight + bias rounded once to the output's dtype.
    x, add_a, add_b: float32 [T, H]; out1, out2 [R, H]; rows: int32 [R] source rows (None: row r).  add_a may be the un-added
    slices of a split product (PartialSums [splits][T][H]): they are added here, in split order."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.is_cuda and x.dim() == 2, "x must be contiguous float32 [T, H]")
    T, H = x.shape
    a_splits = 1
    if isinstance(add_a, PartialSums):
        _need(add_a.rows == T and add_a.cols == H, "an addition's partial sums must match x")
        add_a, a_splits = add_a.data, add_a.splits
        _need(add_a.dtype == torch.float32 and add_a.is_contiguous() and add_a.is_cuda and add_a.numel() >= a_splits * T * H,
              "partial sums must be contiguous float32 [splits][T][H]")
    for t, n in (((add_a if a_splits == 1 else None), "add_a"), (add_b, "add_b")):
        if t is not None:
            _need(t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda and tuple(t.shape) == (T, H), f"{n} must match x")
    _need(add_a is not None or add_b is None, "dyt_norm: a second addition needs a first")
    _need(not replace or add_a is not None, "dyt_norm: nothing to replace x with")
    R, dt = T, 0
    for norm, out in ((first, out1), (second, out2)):
        _need((norm is None) == (out is None), "dyt_norm: every output needs its norm")
        if out is not None:
            _need(out.is_cuda and out.is_contiguous() and out.dim() == 2 and out.shape[1] == H, "out must be contiguous [R, H]")
            _f32(norm.weight, "the norm weight", H)
            _f32(norm.bias, "the norm bias", H)
            R, dt = out.shape[0], _DT[out.dtype]
    if out1 is not None and out2 is not None:
        _need(out1.shape == out2.shape and out1.dtype == out2.dtype, "dyt_norm: the two outputs must agree")
    if rows is not None:
        _i32(rows, "rows", R)
    else:
        _need(R <= T, "x has fewer rows than the output")
    write_back = 1 if (rows is None and add_a is not None) else 0
    _need(write_back or out1 is not None or out2 is not None, "dyt_norm: nothing to do")
    _call("kvcm_dyt_norm", _ptr(x), 0 if replace else 1, _ptr(add_a), a_splits, T * H, _ptr(add_b), _ptr(rows), write_back,
          _ptr(first.weight) if first else 0, _ptr(first.bias) if first else 0, first.alpha if first else 0.0, _ptr(out1),
          _ptr(second.weight) if second else 0, _ptr(second.bias) if second else 0, second.alpha if second else 0.0, _ptr(out2),
          dt, R, H, _stream())


def stream_pack(x, x0, out, add_a=None, add_b=None):
    """out[T, 2H] = [x + add_a + add_b | x0] in out's dtype; x, x0 and the additions float32 [T, H]."""
    T, H = x.shape
    for t, n in ((x, "x"), (x0, "x0"), (add_a, "add_a"), (add_b, "add_b")):
        if t is not None:
            _need(t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda and tuple(t.shape) == (T, H), f"{n} must be float32 [T, H]")
    _need(add_a is not None or add_b is None, "stream_pack: a second addition needs a first")
    _need(out.is_cuda and out.is_contiguous() and tuple(out.shape) == (T, 2 * H), "out must be contiguous [T, 2H]")
    _call("kvcm_stream_pack", _ptr(x), _ptr(add_a), _ptr(add_b), _ptr(x0), _ptr(out), _DT[out.dtype], T, H, _stream())
    return out


def scale_rows(x, factor):
    """x *= factor in place (float32)."""
    _f32(x, "x")
    _call("kvcm_scale_rows", _ptr(x), x.numel(), float(factor), _stream())
    return x


def softcap_rows(x, cap):
    """x <- cap * tanh(x / cap) in place (float32)."""
    _f32(x, "x")
    _need(cap > 0, "softcap_rows: the cap must be positive")
    _call("kvcm_softcap_rows", _ptr(x), x.numel(), float(cap), _stream())
    return x


def head_gate(o, gate, heads, dv, rows=None, per_element=False):
    """o[r, h, :] *= sigmoid(gate[r, h]) in place; o [T, >= heads*dv] in the compute dtype, gate float32 rows of >= heads.
    ``per_element``: a gate logit for every element, o[r, c] *= sigmoid(gate[r, c]), gate rows of >= heads*dv."""
    T = o.shape[0] if rows is None else rows
    _rows2d(o, "o")
    _f32rows(gate, "gate", heads * dv if per_element else heads)
    _need(o.is_cuda and o.shape[1] >= heads * dv and gate.shape[0] >= T and o.shape[0] >= T, "head_gate: shapes do not agree")
    _call("kvcm_head_gate", _ptr(o), _DT[o.dtype], o.stride(0), _ptr(gate), gate.stride(0), T, heads, dv, 1 if per_element else 0, _stream())
    return o


def rms_groups(x, col0, size, groups, weight, eps, rows=None, out=None):
    """On float32 rows: each of ``groups`` stretches of ``size`` columns from col0 on is divided by its root mean
    square (eps inside the root) and multiplied by weight[0 .. size); in place, or with ``out`` (rows of any dtype the
    kernels store, >= groups*size columns) into out from its column 0 on, x left as it is."""
    T = x.shape[0] if rows is None else rows
    _f32rows(x, "x", col0 + size * groups)
    _f32(weight, "weight", size)
    if out is not None:
        _rows2d(out, "out")
        _need(out.is_cuda and out.shape[0] >= T and out.shape[1] >= size * groups, "rms_groups: the output is too small")
    _call("kvcm_rms_groups", _ptr(x), x.stride(0), col0, size, groups, _ptr(weight), float(eps), _ptr(out),
          _DT[out.dtype] if out is not None else 0, out.stride(0) if out is not None else 0, T, _stream())
    return x if out is None else out


class BiasedOutput:
    """A sublayer's output with a bias of its output projection still to be added: ``value`` (a 32-bit tensor or
    PartialSums) + bias[H].  A norm that adds the sublayer's output to the stream adds the bias in the same pass
    (``layernorm_post``); anyone else calls ``materialize()``."""

    def __init__(self, value, bias):
        self.value, self.bias = value, bias

    def materialize(self):
        out = self.value.materialize() if hasattr(self.value, "materialize") else self.value
        out += self.bias      # (a tensor library's routine: not for recorded steps)
        return out


def layernorm_post(x, weight, eps, alpha=1.0, add=None, out=None, rows=None):
    """x <- ln(alpha * x + add) * weight in place, ln(v) = (v - mean) / sqrt(mean of squared deviations + eps), all in
    32-bit; ``add``: a 32-bit tensor like x, PartialSums, a BiasedOutput of either, or None.  ``out`` [R, H] also receives
    the new rows, rounded once to its dtype.  With ``rows`` (int32 [R]) the result of those rows goes to ``out`` only."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.is_cuda and x.dim() == 2, "x must be contiguous float32 [T, H]")
    T, H = x.shape
    _f32(weight, "the norm weight", H)
    bias, a, splits = None, None, 1
    if isinstance(add, BiasedOutput):
        add, bias = add.value, add.bias
        _f32(bias, "the output bias", H)
    if isinstance(add, PartialSums):
        _need(add.rows == T and add.cols == H, "the added product's partial sums must match x")
        a, splits = add.data, add.splits
    elif add is not None:
        _need(add.dtype == torch.float32 and add.is_contiguous() and add.shape == x.shape and add.is_cuda, "the added output must match x")
        a = add
    R = T
    if out is not None:
        _need(out.is_cuda and out.is_contiguous() and out.dim() == 2 and out.shape[1] == H, "out must be contiguous [R, H]")
        R = out.shape[0]
        if rows is not None:
            _i32(rows, "rows", R)
        else:
            _need(R <= T, "x has fewer rows than the output")
    else:
        _need(rows is None, "layernorm_post: gathered rows need an output")
    _call("kvcm_layernorm_post", _ptr(x), _ptr(a), splits, T * H, _ptr(bias), float(alpha), _ptr(weight), _ptr(rows), _ptr(out),
          _DT[out.dtype] if out is not None else 0, R, H, float(eps), _stream())
    return out


def head_norm_store(qkv, q_out, nh, nkv, d, dv, eps, q_weight=None, k_weight=None, bias=None, positions=None, temp_coef=0.0,
                    temp_every=0, values_are_keys=False, slots=None, kcache=None, vcache=None, rows=None):
    """qkv: 32-bit rows [q (nh*d) | k (nkv*d) | v (nkv*dv)] (no v with ``values_are_keys``); ``bias``: a float32 row of
    that layout, added first.  Every q and k head is divided by its own root mean square (eps inside the root) and
    multiplied by ``q_weight`` / ``k_weight`` [d] (None: that kind passes); with ``temp_every`` > 0 the query is then
    multiplied by 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1).  q goes to q_out [T, nh*d], k to its page
    slot, and as values the projection's own or, with ``values_are_keys``, the keys as projected, before their norm."""
    T = q_out.shape[0] if rows is None else rows
    width = (nh + nkv) * d + (0 if values_are_keys else nkv * dv)
    _f32rows(qkv, "qkv", width)
    _rows2d(q_out, "q_out")
    _need(q_out.shape[1] >= nh * d and q_out.is_cuda and qkv.shape[0] >= T, "head_norm_store: shapes do not agree")
    _need(not values_are_keys or d == dv, "head_norm_store: keys can only be values of their own size")
    _f32(q_weight, "q_weight", d)
    _f32(k_weight, "k_weight", d)
    _f32(bias, "bias", width)
    if temp_every > 0:
        _i32(positions, "positions", T)
        _need(positions is not None, "head_norm_store: a temperature by position needs the positions")
    B = 1
    if slots is not None:
        _i32(slots, "slots", T)
        _need(kcache is not None and kcache.dtype == q_out.dtype and kcache.is_contiguous() and kcache.dim() == 4
              and kcache.shape[1] == nkv and kcache.shape[3] == d, "key cache must be [pages, nkv, block_size, d]")
        B = kcache.shape[2]
        _need(vcache is not None and vcache.dtype == q_out.dtype and vcache.is_contiguous()
              and tuple(vcache.shape) == (kcache.shape[0], nkv, dv, B), "value cache must be [pages, nkv, dv, block_size]")
    _call("kvcm_head_norm_store", _ptr(qkv), qkv.stride(0), _ptr(bias), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(positions),
          float(temp_coef), int(temp_every), 1 if values_are_keys else 0, _ptr(slots), _ptr(q_out), _DT[q_out.dtype], q_out.stride(0),
          _ptr(kcache), _ptr(vcache), T, nh, nkv, d, dv, B, _stream())


def gemm_heads(x, w, out, gate=None, rows=None):
    """out[m, h*N + n] = sum_k x[m, h*K + k] * w[h, n, k] for w [heads, N, K]: one small product per head, every head on
    its own stretch of the rows.  x and w in one dtype (float32 gives float32); ``gate`` (float32 rows of >= heads*N):
    the result times sigmoid(gate), element by element, before it is stored."""
    _dev(x, w, out, gate)
    _rows2d(x, "x")
    _rows2d(out, "out")
    _need(w.dim() == 3 and w.is_contiguous() and w.dtype == x.dtype, "gemm_heads: w must be contiguous [heads, N, K] in x's dtype")
    heads, N, K = w.shape
    M = out.shape[0] if rows is None else rows
    _need(x.shape[0] >= M and x.shape[1] >= heads * K and out.shape[1] >= heads * N, "gemm_heads: shapes do not agree")
    _need(x.dtype != torch.float32 or out.dtype == torch.float32, "gemm_heads: float32 operands give a float32 result")
    if gate is not None:
        _f32rows(gate, "gate", heads * N)
        _need(gate.shape[0] >= M, "gemm_heads: the gate has fewer rows than the step")
    _call("kvcm_gemm_heads", _ptr(x), _DT[x.dtype], x.stride(0), _ptr(w), _ptr(out), _DT[out.dtype], out.stride(0), _ptr(gate),
          gate.stride(0) if gate is not None else 0, M, heads, N, K, _stream())
    return out


def act_rows(x, out, activation):
    """out[T, I] = act(x[T, :I]) for 32-bit rows (a tensor, or PartialSums whose slices are added first); act: "silu",
    "relu" or "gelu_tanh"."""
    T, I = out.shape
    _rows2d(out, "out")
    splits, stride = 1, 0
    if isinstance(x, PartialSums):
        _need(x.rows == T and x.cols == I, "act_rows: the partial sums do not match the output")
        x, splits, stride = x.data, x.splits, T * I
        _f32(x, "x", splits * T * I)
        ld = I
    else:
        _f32rows(x, "x", I)
        _need(x.shape[0] >= T, "act_rows: the rows do not agree")
        ld = x.stride(0)
    _need(out.is_cuda, "act_rows: the output must live on the GPU")
    _need(activation in GATE_ACTIVATIONS, f"unknown activation {activation!r} ({sorted(GATE_ACTIVATIONS)})")
    _call("kvcm_act_rows", _ptr(x), ld, splits, stride, _ptr(out), _DT[out.dtype], out.stride(0), T, I, GATE_ACTIVATIONS[activation], _stream())
    return out


def mlstm_scan(q, k, v, gate_in, gate_keep, in_bias, keep_bias, cap, q_scale, coef, n_new, o, s_state, n_state, m_state, step, heads, dk, dv):
    """The matrix memory with exponential gates over the step's runs (csrc/hip/mlstm.hip).  q, k [T, heads*dk], v [T, heads*dv],
    gate_in, gate_keep [T, heads] (projections without biases): 32-bit rows; coef: float32 scratch of 4 T heads values;
    n_new: float32 scratch of seqs heads dk values; states [slots, heads, dk, dv], [slots, heads, dk], [slots, heads]."""
    T = o.shape[0]
    for t, n, c in ((q, "q", heads * dk), (k, "k", heads * dk), (v, "v", heads * dv), (o, "o", heads * dv), (gate_in, "gate_in", heads),
                    (gate_keep, "gate_keep", heads)):
        _f32rows(t, n, c)
        _need(t.shape[0] >= T, f"{n} has too few rows")
    _f32(in_bias, "in_bias", heads)
    _f32(keep_bias, "keep_bias", heads)
    _f32(coef, "coef", 4 * T * heads)
    _f32(n_new, "n_new", step.seqs * heads * dk)
    for t, n, shape in ((s_state, "s_state", (heads, dk, dv)), (n_state, "n_state", (heads, dk)), (m_state, "m_state", (heads,))):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.is_cuda and tuple(t.shape[1:]) == shape, f"{n} must be float32 [slots, {shape}]")
    _call("kvcm_mlstm_scan", _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(gate_in), gate_in.stride(0),
          _ptr(gate_keep), gate_keep.stride(0), _ptr(in_bias), _ptr(keep_bias), float(cap), float(q_scale), _ptr(coef), _ptr(n_new), _ptr(o),
          o.stride(0), _ptr(s_state), _ptr(n_state), _ptr(m_state), _ptr(step.run_start), _ptr(step.seq_start),
          _ptr(step.state_slots), step.seqs, heads, dk, dv, T, int(step.max_run), _stream())
    return o


def moe_route(logits, experts, top, chosen, weight, rows=None, over_chosen=False):
    """chosen[T, top] (int32) and weight[T, top] (float32): the ``top`` experts with the largest softmax scores over all
    ``experts`` of each row's 32-bit router logits, best first, with those scores; ``over_chosen``: with the softmax over
    the chosen logits alone instead (the weights of a row add up to one).  ``logits`` may be PartialSums (a router product
    that was split along K): the slices are added as they are read."""
    T = chosen.shape[0] if rows is None else rows
    splits, stride = 1, 0
    if isinstance(logits, PartialSums):
        _need(logits.rows >= T and logits.cols >= experts, "moe_route: the partial sums do not hold the rows' logits")
        splits, stride, ld, logits = logits.splits, logits.rows * logits.cols, logits.cols, logits.data
        _f32(logits, "logits", splits * stride)
    else:
        _f32rows(logits, "logits", experts)
        _need(logits.shape[0] >= T, "moe_route: fewer rows of logits than rows")
        ld = logits.stride(0)
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and chosen.is_cuda and chosen.shape[1] == top and chosen.shape[0] >= T,
          "chosen must be int32 [T, top]")
    _need(weight.dtype == torch.float32 and weight.is_contiguous() and weight.is_cuda and tuple(weight.shape) == tuple(chosen.shape),
          "weight must be float32 [T, top]")
    _call("kvcm_moe_route", _ptr(logits), ld, splits, stride, experts, top, 1 if over_chosen else 0, _ptr(chosen), _ptr(weight),
          T, _stream())


def moe_table_route(tokens, table, top, chosen, weight, rows=None):
    """chosen[T, top] = table[tokens[T], :top] (int32 table [vocab, >= top] of expert numbers per token id), weight = 1 / top."""
    T = chosen.shape[0] if rows is None else rows
    _i32(tokens, "tokens", T)
    _need(table.dtype == torch.int32 and table.is_cuda and table.dim() == 2 and table.stride(1) == 1 and table.shape[1] >= top,
          "table must be int32 [vocab, >= top]")
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and chosen.is_cuda and chosen.shape[1] == top and chosen.shape[0] >= T,
          "chosen must be int32 [T, top]")
    _need(weight.dtype == torch.float32 and weight.is_contiguous() and weight.is_cuda and tuple(weight.shape) == tuple(chosen.shape),
          "weight must be float32 [T, top]")
    _call("kvcm_moe_table_route", _ptr(tokens), _ptr(table), table.shape[0], table.stride(0), top, _ptr(chosen), _ptr(weight), T, _stream())


def _expert_shapes(w_up, w_down, gated):
    E, rows, K = w_up.shape
    F = rows // 2 if gated else rows
    _need(not gated or (rows % 32 == 0), "gated experts: the interleaved matrix has 2F rows, F a multiple of 16")
    return E, F, K


def moe_rows(h, w_up, w_down, chosen, weight, act, out, gated=False, add=None):
    """out[T, H] (float32) = sum over a row's chosen experts e of weight * W_down[e] square(relu(W_up[e] h)), a row at a
    time, reading only the chosen experts.  h [T, K]; w_up [E, F, K]; w_down [E, H, F]; act: work memory [T * top, F].
    ``gated``: w_up is ``interleave_gate_up`` of the experts' gate and up matrices and the activation is
    silu(W_gate h) * (W_up h).  ``add`` (float32 [T, H]): out = add + the sum."""
    T, K = h.shape
    E, F, _ = _expert_shapes(w_up, w_down, gated)
    H, top = w_down.shape[1], chosen.shape[1]
    if add is not None:
        _need(add.dtype == torch.float32 and add.is_contiguous() and add.is_cuda and tuple(add.shape) == (T, H), "add must be float32 [T, H]")
    _rows2d(h, "h")
    _need(h.is_cuda and h.dtype == w_up.dtype == w_down.dtype == act.dtype, "moe_rows: operands must share one dtype")
    _need(w_up.is_contiguous() and w_down.is_contiguous() and w_up.shape[2] == K and tuple(w_down.shape) == (E, H, F),
          "moe_rows: expert weights must be [E, F, K] ([E, 2F, K] gated) and [E, H, F]")
    _need(act.is_contiguous() and act.shape[0] >= T * top and act.shape[1] == F, "act must be [T * top, F]")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, H), "out must be float32 [T, H]")
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and chosen.shape[0] >= T, "chosen must be int32 [T, top]")
    _need(weight.dtype == torch.float32 and weight.is_contiguous() and tuple(weight.shape) == tuple(chosen.shape), "weight must match chosen")
    _call("kvcm_moe_up", _ptr(h), _DT[h.dtype], h.stride(0), _ptr(w_up), _ptr(chosen), _ptr(act), T, K, F, top, E, 1 if gated else 0, _stream())
    _call("kvcm_moe_down", _ptr(act), _DT[act.dtype], _ptr(w_down), _ptr(chosen), _ptr(weight), _ptr(add), _ptr(out), T, F, H, top, E, _stream())
    return out


def moe_grouped_supported(K, F, E, dtype):
    """Does the grouped form of the routed feed-forward (tiles on the matrix cores) take these sizes?"""
    return dtype == torch.bfloat16 and bool(lib().kvcm_moe_grouped_supported(int(K), int(F), int(E)))


def moe_grouped_tiles(pairs, E):
    """int32 values of work memory that ``moe_grouped`` needs for its list of tiles."""
    return 3 * lib().kvcm_moe_grouped_max_tiles(int(pairs), int(E)) + 1


def moe_grouped(h, w_up, w_down, chosen, weight, order, tiles, act, y, out, gated=False, add=None):
    """As ``moe_rows``, for steps with many rows (bfloat16): the (row, slot) pairs grouped by expert and multiplied in tiles
    on the matrix cores.  Work memory: order int32 [T * top], tiles int32 [moe_grouped_tiles], act [T * top, F],
    y float32 [T * top, H]."""
    T, K = h.shape
    E, F, _ = _expert_shapes(w_up, w_down, gated)
    H, top = w_down.shape[1], chosen.shape[1]
    if add is not None:
        _need(add.dtype == torch.float32 and add.is_contiguous() and add.is_cuda and tuple(add.shape) == (T, H), "add must be float32 [T, H]")
    _rows2d(h, "h")
    _need(h.is_cuda and h.dtype == w_up.dtype == w_down.dtype == act.dtype == torch.bfloat16, "moe_grouped takes bfloat16 operands")
    _need(w_up.is_contiguous() and w_down.is_contiguous() and w_up.shape[2] == K and tuple(w_down.shape) == (E, H, F),
          "moe_grouped: expert weights must be [E, F, K] ([E, 2F, K] gated) and [E, H, F]")
    _need(act.is_contiguous() and act.shape[0] >= T * top and act.shape[1] == F, "act must be [T * top, F]")
    _need(y.dtype == torch.float32 and y.is_contiguous() and y.shape[0] >= T * top and y.shape[1] == H, "y must be float32 [T * top, H]")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, H), "out must be float32 [T, H]")
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous() and chosen.shape[0] >= T, "chosen must be int32 [T, top]")
    _need(weight.dtype == torch.float32 and weight.is_contiguous() and tuple(weight.shape) == tuple(chosen.shape), "weight must match chosen")
    _i32(order, "order", T * top)
    _i32(tiles, "tiles", moe_grouped_tiles(T * top, E))
    _call("kvcm_moe_grouped", _ptr(h), h.stride(0), _ptr(w_up), _ptr(w_down), _ptr(chosen), _ptr(weight), _ptr(order), _ptr(tiles),
          _ptr(act), _ptr(y), _ptr(add), _ptr(out), T, K, F, H, top, E, 1 if gated else 0, _stream())
    return out
