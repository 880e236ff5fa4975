"""MI355X-native token sampling for OpenTail.Stingray: host-side mirror of the engine's sampler
interface over the C ABI of libstingray_sampler.so (include/stingray_sampler.h).

The names follow the reference (src/OpenTail.Stingray.Engine/Sampler.cs): ``SamplingParams`` with the
same fields and defaults, ``Sampler.Sample / Greedy / BuildFilteredDistribution /
SampleWithDistribution / SampleFromProbs / ResampleResidual`` with the same argument meaning and error
behaviour (ArgumentException -> ValueError, ArgumentNullException -> TypeError), and a batched entry,
``SamplerContext.sample_batch``, the sampled sibling of ``IBatchedForwardPass.BatchForwardMultiArgmax``.

Everything here runs on the GPU through the native library; there is no CPU implementation to fall
back to, and loading fails loudly when the library has not been built.
"""
from __future__ import annotations

import ctypes as C
import weakref
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np

__all__ = ["SamplingParams", "Sampler", "SamplerContext", "NativeLibraryError", "load_library", "lib_path"]

_HERE = os.path.dirname(os.path.abspath(__file__))
# STINGRAY_SAMPLER_LIB names another build of the library (the profiling build, say), as the reference's resolver
# probes an override before its default names (src/OpenTail.Stingray.Cuda/CudaLibraryResolver.cs:27-47)
_LIB_PATH = os.environ.get("STINGRAY_SAMPLER_LIB") or os.path.join(_HERE, "lib", "libstingray_sampler.so")

SR_OK = 0
HIP_STREAM_LEGACY = 1  # hipStreamLegacy: the device's default stream, named explicitly
SR_ERR_INVALID_ARGUMENT = 1
SR_ERR_NULL_ARGUMENT = 2
SR_ERR_HIP = 3
SR_ERR_UNSUPPORTED = 4
SR_ERR_OUT_OF_MEMORY = 5
SR_ERR_NO_DEVICE = 6
SR_DTYPE_F32 = 0
SR_DTYPE_BF16 = 1
SR_ROW_HAS_LOGIT_BIAS = 1
SR_ROW_DRAFT_FROM_LOOKUP = 2
SR_OUT_PATH_GREEDY = 1
SR_OUT_PATH_TOPK_FAST = 2
SR_OUT_PATH_FULL_VOCAB = 4
SR_OUT_DEGENERATE = 8
SR_OUT_AMBIGUOUS = 16
SR_OUT_ROW_UNSUPPORTED = 1 << 31

# every symbol include/stingray_sampler.h declares
EXPORTED_SYMBOLS = [
    "sr_create", "sr_destroy", "sr_bind_thread", "sr_set_stream", "sr_use_own_stream", "sr_synchronize", "sr_last_error",
    "sr_version", "sr_batch_create", "sr_batch_destroy", "sr_batch_upload", "sr_batch_set_uniforms",
    "sr_batch_append_tokens", "sr_batch_append_tokens_masks", "sr_batch_upload_mask_ids", "sr_mask_register",
    "sr_mask_release", "sr_mask_and", "sr_pack_allow_mask_launch",
    "sr_sample_launch", "sr_resample_rows_launch", "sr_sample_batch", "sr_argmax_rows_launch", "sr_argmax_rows_launch_noalloc",
    "sr_argmax_rows",
    "sr_build_distribution_launch", "sr_sample_with_distribution_launch", "sr_sample_from_probs_launch",
    "sr_resample_residual_launch", "sr_spec_verify_launch", "sr_mtp_verify_launch", "sr_pack_allow_mask",
    "sr_build_distribution", "sr_sample_with_distribution", "sr_sample_from_probs", "sr_resample_residual",
]


class NativeLibraryError(RuntimeError):
    pass


class RowParams(C.Structure):
    """sr_row_params"""

    _fields_ = [
        ("temperature", C.c_float),
        ("top_k", C.c_int32),
        ("top_p", C.c_float),
        ("min_p", C.c_float),
        ("repetition_penalty", C.c_float),
        ("repeat_last_n", C.c_int32),
        ("presence_penalty", C.c_float),
        ("frequency_penalty", C.c_float),
        ("spec_draft_p_min", C.c_float),
        ("flags", C.c_uint32),
    ]


@dataclass
class SamplingParams:
    """Sampler.cs:648-813 -- the fields the sampler reads, same names and defaults."""

    Temperature: float = 1.0
    TopK: int = 0
    TopP: float = 1.0
    MinP: float = 0.0
    RepetitionPenalty: float = 1.0
    RepeatLastN: int = 64
    PresencePenalty: float = 0.0
    FrequencyPenalty: float = 0.0
    LogitBias: Optional[Dict[int, float]] = None
    PreviousTokens: Optional[Sequence[int]] = None
    SpecDraftPMin: float = 1.0
    # not a field of the reference's SamplingParams: the step's `usedPld` (SpeculativeDecoder.cs:488-501), which the
    # accept loop reads beside them (:538, :549)
    SpecDraftFromLookup: bool = False

    @property
    def HasHistoryPenalty(self) -> bool:
        return self.RepetitionPenalty != 1.0 or self.PresencePenalty != 0.0 or self.FrequencyPenalty != 0.0

    def to_row(self) -> RowParams:
        return RowParams(self.Temperature, self.TopK, self.TopP, self.MinP, self.RepetitionPenalty,
                         self.RepeatLastN, self.PresencePenalty, self.FrequencyPenalty, self.SpecDraftPMin,
                         (SR_ROW_HAS_LOGIT_BIAS if self.LogitBias else 0)
                         | (SR_ROW_DRAFT_FROM_LOOKUP if self.SpecDraftFromLookup else 0))


_lib = None


def lib_path() -> str:
    return _LIB_PATH


def load_library():
    """Loads libstingray_sampler.so. Raises NativeLibraryError when it has not been built
    (python -m opentail.stingray_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise NativeLibraryError(
            f"{_LIB_PATH} is missing: build it with `python -m opentail.stingray_amd.build` "
            "(hipcc, gfx950). There is no CPU fallback.")
    # torch brings its own copy of the HIP runtime.  It has to be the first one in the process: with the system's
    # runtime loaded before it (by this library), torch finds no GPU afterwards.  Loaded second, this library binds
    # to the runtime that is already there.
    try:
        import torch  # noqa: F401
    except ImportError:  # pragma: no cover - the mirror allocates through torch, the library itself does not need it
        pass
    try:
        L = C.CDLL(_LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the host
        raise NativeLibraryError(f"cannot load {_LIB_PATH}: {e}") from e
    vp, i32, i64, u32p, i32p, f32p, f64p = (C.c_void_p, C.c_int32, C.c_int64, C.POINTER(C.c_uint32),
                                             C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_double))
    rpp = C.POINTER(RowParams)
    L.sr_create.argtypes = [C.c_int, C.POINTER(vp)]
    L.sr_destroy.argtypes = [vp]
    L.sr_destroy.restype = None
    L.sr_bind_thread.argtypes = [vp]
    L.sr_set_stream.argtypes = [vp, vp]
    L.sr_use_own_stream.argtypes = [vp]
    L.sr_synchronize.argtypes = [vp]
    L.sr_last_error.argtypes = [vp]
    L.sr_last_error.restype = C.c_char_p
    L.sr_version.restype = C.c_char_p
    L.sr_batch_create.argtypes = [vp, C.POINTER(vp)]
    L.sr_batch_destroy.argtypes = [vp]
    L.sr_batch_destroy.restype = None
    L.sr_batch_upload.argtypes = [vp, i32, i32, rpp, i32p, i32p, i32p, f32p, i32p, u32p, i64,
                                  C.POINTER(C.c_uint8), f64p, i32]
    L.sr_batch_set_uniforms.argtypes = [vp, f64p]
    L.sr_batch_append_tokens.argtypes = [vp, i32p, f64p]
    L.sr_batch_append_tokens_masks.argtypes = [vp, i32p, f64p, i32p]
    L.sr_batch_upload_mask_ids.argtypes = [vp, i32, i32, rpp, i32p, i32p, i32p, f32p, i32p, i32p, f64p, i32]
    L.sr_mask_register.argtypes = [vp, vp, C.c_int, i32, i32p]
    L.sr_mask_release.argtypes = [vp, i32]
    L.sr_mask_and.argtypes = [vp, i32p, i32, i32p]
    L.sr_pack_allow_mask_launch.argtypes = [vp, vp, C.c_int, i32, i32, i64, vp, i64]
    L.sr_sample_launch.argtypes = [vp, vp, vp, C.c_int, i64, vp, vp]
    L.sr_resample_rows_launch.argtypes = [vp, vp, vp, C.c_int, i64, i32p, i32, vp, vp]
    L.sr_sample_batch.argtypes = [vp, vp, C.c_int, C.c_int, i32, i32, i64, rpp, i32p, i32p, i32p, f32p, i32p,
                                  u32p, i64, C.POINTER(C.c_uint8), f64p, i32p, u32p]
    L.sr_argmax_rows_launch.argtypes = [vp, vp, C.c_int, i32, i32, i64, vp, vp]
    L.sr_argmax_rows_launch_noalloc.argtypes = [vp, vp, C.c_int, i32, i32, i64, vp, vp]
    L.sr_argmax_rows.argtypes = [vp, vp, C.c_int, C.c_int, i32, i32, i64, i32p, f32p]
    L.sr_build_distribution_launch.argtypes = [vp, vp, vp, C.c_int, i64, vp, i64, i32]
    L.sr_sample_with_distribution_launch.argtypes = [vp, vp, vp, C.c_int, i64, vp, i64, i32, vp]
    L.sr_sample_from_probs_launch.argtypes = [vp, vp, i32, i32, i64, f64p, vp]
    L.sr_resample_residual_launch.argtypes = [vp, vp, i32, i64, vp, i32, i64, i32, f64p, vp]
    L.sr_spec_verify_launch.argtypes = [vp, vp, vp, vp, vp, i32, vp, vp]
    L.sr_mtp_verify_launch.argtypes = [vp, vp, i32, i32, i64, vp, C.c_float, vp, vp, vp]
    L.sr_pack_allow_mask.argtypes = [f32p, i32, u32p]
    _lib = L
    return L


def _ptr(a: Optional[np.ndarray], ctype):
    return None if a is None else a.ctypes.data_as(C.POINTER(ctype))


def pack_allow_mask(allowed: np.ndarray) -> np.ndarray:
    """bool[rows, vocab] (or [vocab]) -> uint32 words, bit (i & 31) of word (i >> 5)."""
    a = np.asarray(allowed, dtype=bool)
    one = a.ndim == 1
    a = np.atleast_2d(a)
    rows, vocab = a.shape
    nw = (vocab + 31) // 32
    padded = np.zeros((rows, nw * 32), dtype=bool)
    padded[:, :vocab] = a
    words = np.packbits(padded.reshape(rows, nw, 32), axis=-1, bitorder="little").view(np.uint32).reshape(rows, nw)
    return words[0] if one else words


class _Batch:
    def __init__(self, ctx: "SamplerContext"):
        self.ctx = ctx
        self.h = C.c_void_p()
        ctx._check(ctx.L.sr_batch_create(ctx.h, C.byref(self.h)))
        ctx._batches.add(self)  # a batch must not outlive its context: the context closes what is left
        self.rows = 0
        self.vocab = 0

    def upload(self, params: Sequence[SamplingParams], vocab: int, uniforms=None, allow_mask=None,
               mask_active=None, uniforms_per_row: Optional[int] = None, mask_ids=None):
        """mask_ids: per row the id of a registered allow-mask (SamplerContext.register_mask), -1 for none, instead
        of allow_mask / mask_active."""
        rows = len(params)
        arr = (RowParams * max(rows, 1))()
        hist: List[int] = []
        hoff = [0]
        bids: List[int] = []
        bvals: List[float] = []
        boff = [0]
        for i, p in enumerate(params):
            arr[i] = p.to_row()
            if p.PreviousTokens is not None:
                hist.extend(int(t) for t in p.PreviousTokens)
            hoff.append(len(hist))
            if p.LogitBias:
                for k_, v_ in p.LogitBias.items():
                    bids.append(int(k_))
                    bvals.append(float(v_))
            boff.append(len(bids))
        h_ids = np.asarray(hist, dtype=np.int32) if hist else None
        h_off = np.asarray(hoff, dtype=np.int32)
        b_ids = np.asarray(bids, dtype=np.int32) if bids else None
        b_vals = np.asarray(bvals, dtype=np.float32) if bids else None
        b_off = np.asarray(boff, dtype=np.int32) if bids else None
        m = None
        stride = 0
        act = None
        if allow_mask is not None:
            m = np.ascontiguousarray(np.asarray(allow_mask, dtype=np.uint32))
            assert m.ndim == 2 and m.shape[0] == rows
            stride = m.shape[1]
            if mask_active is not None:
                act = np.ascontiguousarray(np.asarray(mask_active, dtype=np.uint8))
        u = None
        upr = 0
        if uniforms is not None and rows > 0:
            u = np.ascontiguousarray(np.asarray(uniforms, dtype=np.float64)).reshape(rows, -1)
            upr = u.shape[1] if uniforms_per_row is None else uniforms_per_row
        self._packed = (rows, vocab, arr, h_ids, h_off, b_ids, b_vals, b_off, m, stride, act, u, upr)
        self.rows, self.vocab = rows, vocab
        if mask_ids is not None:
            assert allow_mask is None
            ids = np.ascontiguousarray(np.asarray(mask_ids, dtype=np.int32))
            assert ids.shape == (rows,)
            self.ctx._check(self.ctx.L.sr_batch_upload_mask_ids(
                self.h, rows, vocab, arr, _ptr(h_ids, C.c_int32), _ptr(h_off, C.c_int32), _ptr(b_ids, C.c_int32),
                _ptr(b_vals, C.c_float), _ptr(b_off, C.c_int32), _ptr(ids, C.c_int32), _ptr(u, C.c_double), upr))
            return self
        return self.reupload()

    def reupload(self):
        """sr_batch_upload once more with the arrays of the last upload(): what a decode step costs the host beyond
        gathering its parameters."""
        rows, vocab, arr, h_ids, h_off, b_ids, b_vals, b_off, m, stride, act, u, upr = self._packed
        self.ctx._check(self.ctx.L.sr_batch_upload(
            self.h, rows, vocab, arr, _ptr(h_ids, C.c_int32), _ptr(h_off, C.c_int32),
            _ptr(b_ids, C.c_int32), _ptr(b_vals, C.c_float), _ptr(b_off, C.c_int32),
            _ptr(m, C.c_uint32), stride, _ptr(act, C.c_uint8), _ptr(u, C.c_double), upr))
        return self

    def append_tokens(self, tokens, uniforms=None, mask_ids=None):
        """sr_batch_append_tokens: one more token per row (negative = none) at the end of the histories of the last
        upload(), and optionally the uniforms of the next step.  mask_ids (batches uploaded with mask ids): the
        registered allow-mask of every row for the next step (sr_batch_append_tokens_masks)."""
        t = np.ascontiguousarray(np.asarray(tokens, dtype=np.int32))
        assert t.shape == (self.rows,)
        u = None
        if uniforms is not None:
            u = np.ascontiguousarray(np.asarray(uniforms, dtype=np.float64))
        if mask_ids is not None:
            ids = np.ascontiguousarray(np.asarray(mask_ids, dtype=np.int32))
            assert ids.shape == (self.rows,)
            self.ctx._check(self.ctx.L.sr_batch_append_tokens_masks(self.h, _ptr(t, C.c_int32), _ptr(u, C.c_double),
                                                                    _ptr(ids, C.c_int32)))
            return self
        self.ctx._check(self.ctx.L.sr_batch_append_tokens(self.h, _ptr(t, C.c_int32), _ptr(u, C.c_double)))
        return self

    def set_uniforms(self, uniforms):
        u = np.ascontiguousarray(np.asarray(uniforms, dtype=np.float64))
        self.ctx._check(self.ctx.L.sr_batch_set_uniforms(self.h, _ptr(u, C.c_double)))

    def close(self):
        if self.h:
            self.ctx._batches.discard(self)
            if self.ctx.h:
                self.ctx.L.sr_batch_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


class SamplerContext:
    """One native context (one engine). Tensors are torch CUDA tensors; torch is only the allocator."""

    def __init__(self, device: int = 0, use_torch_stream: bool = True):
        self.L = load_library()
        self.h = C.c_void_p()
        self._batches = weakref.WeakSet()
        rc = self.L.sr_create(device, C.byref(self.h))
        if rc == SR_ERR_NO_DEVICE:
            raise NativeLibraryError("no HIP device: the sampler has no CPU path")
        if rc != SR_OK:
            raise NativeLibraryError(f"sr_create failed: {rc}")
        self.device = device
        if use_torch_stream:
            import torch

            # torch's current stream; its default stream has the handle 0, which is HIP's default stream here too
            handle = torch.cuda.current_stream(device).cuda_stream
            self._check(self.L.sr_set_stream(self.h, C.c_void_p(handle)))

    # -- plumbing ------------------------------------------------------------------------------
    def _check(self, rc: int):
        if rc == SR_OK:
            return
        msg = self.L.sr_last_error(self.h).decode()
        if rc == SR_ERR_INVALID_ARGUMENT:
            raise ValueError(msg)           # ArgumentException
        if rc == SR_ERR_NULL_ARGUMENT:
            raise TypeError(msg)            # ArgumentNullException
        if rc == SR_ERR_UNSUPPORTED:
            raise NotImplementedError(msg)
        raise RuntimeError(f"native sampler error {rc}: {msg}")

    def set_stream(self, stream_handle: Optional[int]):
        """A hipStream_t handle (0 = the device's default stream); None = the context's own stream."""
        if stream_handle is None:
            self._check(self.L.sr_use_own_stream(self.h))
        else:
            self._check(self.L.sr_set_stream(self.h, C.c_void_p(stream_handle)))

    def synchronize(self):
        self._check(self.L.sr_synchronize(self.h))

    def new_batch(self) -> _Batch:
        return _Batch(self)

    def register_mask(self, words, vocab: int) -> int:
        """sr_mask_register: packed allow-bits (numpy uint32 array, or a CUDA int32/uint32 tensor) -> mask id."""
        out = C.c_int32(-1)
        if isinstance(words, np.ndarray):
            w = np.ascontiguousarray(words, dtype=np.uint32)
            assert w.size >= (vocab + 31) // 32
            self._check(self.L.sr_mask_register(self.h, w.ctypes.data_as(C.c_void_p), 0, vocab, C.byref(out)))
        else:
            assert words.is_cuda and words.numel() >= (vocab + 31) // 32
            self._check(self.L.sr_mask_register(self.h, C.c_void_p(words.data_ptr()), 1, vocab, C.byref(out)))
        return int(out.value)

    def mask_and(self, mask_ids) -> int:
        """sr_mask_and: the registered intersection of the given masks (-1 entries skipped), or -1 when nothing is
        left to intersect or the intersection allows no token (the row then goes unmasked)."""
        ids = np.ascontiguousarray(np.asarray(mask_ids, dtype=np.int32))
        out = C.c_int32(-1)
        self._check(self.L.sr_mask_and(self.h, _ptr(ids, C.c_int32), int(ids.size), C.byref(out)))
        return int(out.value)

    def release_mask(self, mask_id: int) -> None:
        self._check(self.L.sr_mask_release(self.h, int(mask_id)))

    def pack_allow_mask_launch(self, masked_logits):
        """Packed allow-bits [rows, ceil(vocab / 32)] (a CUDA int32 tensor holding the uint32 words) of masked rows
        that are on the device: bit set iff the element is not -inf."""
        import torch

        rows, vocab = masked_logits.shape
        out = torch.zeros((rows, (vocab + 31) // 32), dtype=torch.int32, device=masked_logits.device)
        self._check(self.L.sr_pack_allow_mask_launch(
            self.h, C.c_void_p(masked_logits.data_ptr()), self._dtype_of(masked_logits), rows, vocab,
            self._row_stride(masked_logits), C.c_void_p(out.data_ptr()), out.shape[1]))
        return out

    def close(self):
        if self.h:
            for b in list(self._batches):
                b.close()
            self.L.sr_destroy(self.h)
            self.h = C.c_void_p()

    @staticmethod
    def _row_stride(t) -> int:
        """Row stride in elements; a single-row tensor may carry a meaningless stride."""
        rows, vocab = t.shape[0], t.shape[-1]
        assert t.stride(-1) == 1 or vocab <= 1, "rows must be contiguous"
        return t.stride(0) if rows > 1 else max(int(t.stride(0)), vocab)

    @staticmethod
    def _dtype_of(t) -> int:
        import torch

        if t.dtype == torch.float32:
            return SR_DTYPE_F32
        if t.dtype == torch.bfloat16:
            return SR_DTYPE_BF16
        raise ValueError(f"unsupported logits dtype {t.dtype}")

    # -- batched entry points -------------------------------------------------------------------
    def sample_launch(self, batch: _Batch, logits, out_tokens, out_flags=None):
        """Async: logits [rows, vocab] CUDA tensor (row stride in elements), outputs CUDA int32."""
        assert logits.is_cuda and out_tokens.is_cuda
        self._check(self.L.sr_sample_launch(
            self.h, batch.h, C.c_void_p(logits.data_ptr()), self._dtype_of(logits), self._row_stride(logits),
            C.c_void_p(out_tokens.data_ptr()), C.c_void_p(out_flags.data_ptr() if out_flags is not None else 0)))

    def resample_rows_launch(self, batch: _Batch, logits, rows, out_tokens, out_flags=None):
        """Async: SampleTopK by device-wide sorts for the given rows of the batch (those a launch flagged
        SR_OUT_ROW_UNSUPPORTED); same tensors as sample_launch."""
        r = np.ascontiguousarray(rows, dtype=np.int32)
        self._check(self.L.sr_resample_rows_launch(
            self.h, batch.h, C.c_void_p(logits.data_ptr()), self._dtype_of(logits), self._row_stride(logits),
            r.ctypes.data_as(C.POINTER(C.c_int32)), int(r.size),
            C.c_void_p(out_tokens.data_ptr()), C.c_void_p(out_flags.data_ptr() if out_flags is not None else 0)))

    def sample_batch(self, logits, params: Sequence[SamplingParams], uniforms, allow_mask=None, mask_active=None,
                     return_flags: bool = False):
        """Sampler.Sample for every row (preceded by the row's mask). logits: CUDA tensor [rows, vocab].
        Returns numpy int32 tokens (and flags)."""
        import torch

        rows, vocab = logits.shape
        batch = self.new_batch().upload(params, vocab, uniforms, allow_mask, mask_active)
        toks = torch.empty(rows, dtype=torch.int32, device=logits.device)
        flags = torch.zeros(rows, dtype=torch.int32, device=logits.device)
        self.sample_launch(batch, logits, toks, flags)
        self.synchronize()
        torch.cuda.synchronize()
        redo = np.nonzero(flags.cpu().numpy().view(np.uint32) & np.uint32(SR_OUT_ROW_UNSUPPORTED))[0]
        if redo.size:  # rows that overflowed the selection kernel's row tail: as sr_sample_batch does
            self.resample_rows_launch(batch, logits, redo, toks, flags)
            self.synchronize()
            torch.cuda.synchronize()
        batch.close()
        t = toks.cpu().numpy()
        return (t, flags.cpu().numpy().view(np.uint32)) if return_flags else t

    def argmax_rows(self, logits, out=None, noalloc=False):
        """(int Token, float Logit)[] per row -- BatchForwardMultiArgmax's result shape.  out=(idx, val) device
        tensors to write into; noalloc=True goes through the entry point that allocates no device memory."""
        import torch

        rows, vocab = logits.shape
        idx, val = out if out is not None else (torch.empty(rows, dtype=torch.int32, device=logits.device),
                                                torch.empty(rows, dtype=torch.float32, device=logits.device))
        fn = self.L.sr_argmax_rows_launch_noalloc if noalloc else self.L.sr_argmax_rows_launch
        self._check(fn(
            self.h, C.c_void_p(logits.data_ptr()), self._dtype_of(logits), rows, vocab,
            self._row_stride(logits) if rows > 0 and vocab > 0 else vocab, C.c_void_p(idx.data_ptr()), C.c_void_p(val.data_ptr())))
        self.synchronize()
        return idx.cpu().numpy(), val.cpu().numpy()

    def build_distribution(self, logits, params: Sequence[SamplingParams], probs_len: Optional[int] = None,
                           allow_mask=None, mask_active=None):
        import torch

        rows, vocab = logits.shape
        n = vocab if probs_len is None else probs_len
        batch = self.new_batch().upload(params, vocab, None, allow_mask, mask_active)
        out = torch.zeros((rows, n), dtype=torch.float32, device=logits.device)
        try:
            self._check(self.L.sr_build_distribution_launch(
                self.h, batch.h, C.c_void_p(logits.data_ptr()), self._dtype_of(logits), self._row_stride(logits),
                C.c_void_p(out.data_ptr()), self._row_stride(out), n))
            self.synchronize()
        finally:
            batch.close()
        return out

    def sample_with_distribution(self, logits, params: Sequence[SamplingParams], uniforms):
        import torch

        rows, vocab = logits.shape
        batch = self.new_batch().upload(params, vocab, uniforms)
        out = torch.zeros((rows, vocab), dtype=torch.float32, device=logits.device)
        toks = torch.empty(rows, dtype=torch.int32, device=logits.device)
        try:
            self._check(self.L.sr_sample_with_distribution_launch(
                self.h, batch.h, C.c_void_p(logits.data_ptr()), self._dtype_of(logits), self._row_stride(logits),
                C.c_void_p(out.data_ptr()), self._row_stride(out), vocab, C.c_void_p(toks.data_ptr())))
            self.synchronize()
        finally:
            batch.close()
        return toks.cpu().numpy(), out

    def sample_with_distribution_launch(self, batch: _Batch, logits, out_probs, out_tokens):
        """Async: the draft side of StepSampled (SpeculativeDecoder.cs:509-513): distributions and drawn tokens of
        every row stay on the device (out_probs [rows, vocab] fp32, out_tokens [rows] int32, CUDA tensors)."""
        vocab = logits.shape[-1]
        self._check(self.L.sr_sample_with_distribution_launch(
            self.h, batch.h, C.c_void_p(logits.data_ptr()), self._dtype_of(logits), self._row_stride(logits),
            C.c_void_p(out_probs.data_ptr()), self._row_stride(out_probs), vocab, C.c_void_p(out_tokens.data_ptr())))

    def spec_verify_launch(self, batch: _Batch, target_logits, draft_probs, draft_tokens, out_accepted, out_tokens):
        """Async: sr_spec_verify_launch over device tensors (target [rows, L+1, V], q [rows, L, V], tokens [rows, L])."""
        L = target_logits.shape[1] - 1
        self._check(self.L.sr_spec_verify_launch(
            self.h, batch.h, C.c_void_p(target_logits.data_ptr()),
            C.c_void_p(None if draft_probs is None else draft_probs.data_ptr()),
            C.c_void_p(draft_tokens.data_ptr()), L, C.c_void_p(out_accepted.data_ptr()),
            C.c_void_p(out_tokens.data_ptr())))

    def sample_from_probs(self, probs, uniforms):
        import torch

        rows, vocab = probs.shape
        u = None if uniforms is None else np.ascontiguousarray(np.asarray(uniforms, dtype=np.float64))
        toks = torch.empty(rows, dtype=torch.int32, device=probs.device)
        self._check(self.L.sr_sample_from_probs_launch(
            self.h, C.c_void_p(probs.data_ptr()), rows, vocab, self._row_stride(probs), _ptr(u, C.c_double),
            C.c_void_p(toks.data_ptr())))
        self.synchronize()
        return toks.cpu().numpy()

    def resample_residual(self, p, q, uniforms):
        import torch

        rows = p.shape[0]
        u = None if uniforms is None else np.ascontiguousarray(np.asarray(uniforms, dtype=np.float64))
        toks = torch.empty(rows, dtype=torch.int32, device=p.device)
        self._check(self.L.sr_resample_residual_launch(
            self.h, C.c_void_p(p.data_ptr()), p.shape[1], self._row_stride(p), C.c_void_p(q.data_ptr()), q.shape[1],
            self._row_stride(q), rows, _ptr(u, C.c_double), C.c_void_p(toks.data_ptr())))
        self.synchronize()
        return toks.cpu().numpy()

    def spec_verify(self, target_logits, draft_probs, draft_tokens, params: Sequence[SamplingParams], uniforms):
        """target_logits [rows, L+1, V], draft_probs [rows, L, V], draft_tokens [rows, L] (CUDA);
        uniforms [rows, L+1]. Returns (accepted[rows], tokens[rows, L+1])."""
        import torch

        rows, lp1, vocab = target_logits.shape
        L = lp1 - 1
        batch = self.new_batch().upload(params, vocab, uniforms, uniforms_per_row=L + 1)
        acc = torch.empty(rows, dtype=torch.int32, device=target_logits.device)
        toks = torch.empty((rows, L + 1), dtype=torch.int32, device=target_logits.device)
        try:
            self._check(self.L.sr_spec_verify_launch(
                self.h, batch.h, C.c_void_p(target_logits.data_ptr()),
            C.c_void_p(None if draft_probs is None else draft_probs.data_ptr()),
                C.c_void_p(draft_tokens.data_ptr()), L, C.c_void_p(acc.data_ptr()), C.c_void_p(toks.data_ptr())))
            self.synchronize()
        finally:
            batch.close()
        return acc.cpu().numpy(), toks.cpu().numpy()

    def mtp_verify(self, logits, draft_tokens, p_min: float):
        import torch

        rows, vocab = logits.shape
        am = torch.empty(rows, dtype=torch.int32, device=logits.device)
        ok = torch.empty(rows, dtype=torch.int32, device=logits.device)
        pr = torch.empty(rows, dtype=torch.float32, device=logits.device)
        self._check(self.L.sr_mtp_verify_launch(
            self.h, C.c_void_p(logits.data_ptr()), rows, vocab, self._row_stride(logits),
            C.c_void_p(draft_tokens.data_ptr()), p_min, C.c_void_p(am.data_ptr()), C.c_void_p(ok.data_ptr()),
            C.c_void_p(pr.data_ptr())))
        self.synchronize()
        return am.cpu().numpy(), ok.cpu().numpy().astype(bool), pr.cpu().numpy()


_default_ctx: Optional[SamplerContext] = None


def _ctx() -> SamplerContext:
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = SamplerContext(0)
    return _default_ctx


def _as_cuda_row(x):
    import torch

    if isinstance(x, torch.Tensor):
        t = x if x.is_cuda else x.cuda()
        return t.reshape(1, -1)
    return torch.from_numpy(np.ascontiguousarray(np.asarray(x, dtype=np.float32))).cuda().reshape(1, -1)


class Sampler:
    """The static class of Sampler.cs, one row per call. ``rng`` is any object with NextDouble()
    (System.Random's method); a number draws are taken from it exactly when the reference would."""

    @staticmethod
    def Greedy(logits) -> int:                                         # Sampler.cs:442-446
        row = _as_cuda_row(logits)
        if row.shape[1] == 0:
            return 0
        idx, _ = _ctx().argmax_rows(row)
        return int(idx[0])

    @staticmethod
    def Sample(logits, p: SamplingParams, rng=None) -> int:            # Sampler.cs:17-102
        row = _as_cuda_row(logits)
        greedy = p.Temperature <= 0.0
        u = None if greedy else [rng.NextDouble()]
        return int(_ctx().sample_batch(row, [p], u)[0])

    @staticmethod
    def BuildFilteredDistribution(logits, p: SamplingParams, probs_len: Optional[int] = None):  # :118-163
        row = _as_cuda_row(logits)
        return _ctx().build_distribution(row, [p], probs_len)[0]

    @staticmethod
    def SampleWithDistribution(logits, p: SamplingParams, rng=None):   # Sampler.cs:172-187
        row = _as_cuda_row(logits)
        u = [0.0] if p.Temperature <= 0.0 else [rng.NextDouble()]
        toks, probs = _ctx().sample_with_distribution(row, [p], u)
        return int(toks[0]), probs[0]

    @staticmethod
    def SampleFromProbs(probs, rng) -> int:                            # Sampler.cs:195-199
        if rng is None:
            raise TypeError("rng")
        return int(_ctx().sample_from_probs(_as_cuda_row(probs), [rng.NextDouble()])[0])

    @staticmethod
    def ResampleResidual(p, q, rng) -> int:                            # Sampler.cs:587-618
        if rng is None:
            raise TypeError("rng")
        pr, qr = _as_cuda_row(p), _as_cuda_row(q)
        if pr.shape[1] != qr.shape[1]:
            raise ValueError(f"p and q must have equal length ({pr.shape[1]} vs {qr.shape[1]}).")
        return int(_ctx().resample_residual(pr, qr, [rng.NextDouble()])[0])
