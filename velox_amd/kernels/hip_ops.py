"""Python face of the HIP kernels: shape and dtype checks on the host, then a C call on the current stream.

Every kernel the model calls goes through one method of :class:`HipOps`.  The methods check
what the kernels and their launch grids assume (devices, dtypes, contiguity, alignment, sizes)
before launching, because a kernel that reads out of bounds takes the whole GPU down.  There
is no fallback: without a GPU, without hipcc or without the libraries, loading fails.

Matrix products: a float32 run uses the exact FMA kernel (``gemm.hip``); so does any operand mix
a library has no call for.  bfloat16 x bfloat16 products go to the library behind
``torch.nn.functional.linear`` (hipBLASLt), as the reference uses cuBLAS through ``nn.Linear``
(reference ``src/self_attention.py:48,90``, ``src/mlp.py:13,15``).
"""
from __future__ import annotations

import ctypes
import logging
import os
import tempfile
from typing import Tuple, Dict, Optional

import torch

from ..parts.base import DeferredNorm, ResidualSink
from . import build

logger = logging.getLogger(__name__)

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    if dtype not in _DTYPE_CODE:
        raise KernelError(f"kernels take float32 or bfloat16, got {dtype}")
    return _DTYPE_CODE[dtype]


def _ptr(t: Optional[torch.Tensor]):
    return _P(0) if t is None else _P(t.data_ptr())


class PreparedWeight:
    """A ``[N, K]`` weight together with the copies of it that the decode-sized products read (``HipOps.prepare_weight``).
    The part that owns the weight owns this; it stands wherever the weight stands in ``linear``, ``linear_silu_mul`` and
    ``qkv_rope_write``.  ``copies``: 1 and 2 = ``pack_rows`` of the weight as one matrix or as two stacked ones,
    ``"rotary"`` = the copy in the row order of ``qkv_rope_write``."""

    def __init__(self, weight: torch.Tensor) -> None:
        self.weight = weight
        self.version = weight._version
        self.copies: Dict[object, torch.Tensor] = {}

    @property
    def shape(self):
        return self.weight.shape

    @property
    def dtype(self):
        return self.weight.dtype

    def copy(self, key=1) -> Optional[torch.Tensor]:
        if self.weight._version != self.version:
            raise KernelError("a weight was changed in place after the kernels prepared their copies of it; prepare it again")
        return self.copies.get(key)


def _weight_of(weight) -> Tuple[torch.Tensor, Optional[PreparedWeight]]:
    if isinstance(weight, PreparedWeight):
        return weight.weight, weight
    return weight, None


class HipOps:
    name = "hip-gfx950"

    def __init__(self, device) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("the HIP kernels need a GPU (device 'cuda'); there is no CPU path")
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        arch = torch.cuda.get_device_properties(self.device).gcnArchName.split(":")[0]
        if arch != build.ARCH:
            raise KernelError(f"the kernels are built for {build.ARCH}; this GPU is {arch}")
        self._core = ctypes.CDLL(build.ensure_core())
        self._attention: Dict[int, ctypes.CDLL] = {}
        self._declare_core()
        self.num_cus = torch.cuda.get_device_properties(self.device).multi_processor_count
        self.use_library_gemm = True
        self.use_skinny_gemm = True
        self.pack_decode_weights = True
        self.fuse_residual_norm = True
        self._mm_out_dtype_ok: Optional[bool] = None
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)

    # -- loading --------------------------------------------------------------------------------
    def _declare_core(self) -> None:
        c = self._core
        c.velox_embed.argtypes = [_P, _P, _P, _I, _I, _I, _I, _P]
        c.velox_place_tokens.argtypes = [_P, _P, _P, _P, _I, _I, _I, _P]
        c.velox_add_rmsnorm.argtypes = [_P, _P, _P, _P, _P, _I, _I, _F, _I, _I, _I, ctypes.c_longlong, _P]
        c.velox_skinny_qkv_rotary_bf16.argtypes = [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _I, _F, _F, _I, _P]
        c.velox_silu_mul.argtypes = [_P, _P, _I, _I, _I, _P]
        c.velox_rope_kv_write.argtypes = [_P, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]
        c.velox_rope_kv_write_partial_bf16.argtypes = [_P, _P, _I, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]
        c.velox_rope_kv_write_partial_bf16.restype = _I
        c.velox_gemm_fma.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]
        c.velox_skinny_gemm_bf16.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _I, _F, _F, _I, _P]
        c.velox_skinny_residual_norm_bf16.argtypes = [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _P]
        c.velox_skinny_residual_norm_bf16.restype = _I
        c.velox_row_scale_apply.argtypes = [_P, _P, _I, _F, _F, _P, _I, _I, _P]
        c.velox_skinny_gemm_bf16.restype = _I
        c.velox_skinny_gemm_glu_bf16.argtypes = [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _I, _F, _F, _I, _P, _P]
        c.velox_skinny_gemm_glu_bf16.restype = _I
        c.velox_skinny_glu_rows_bf16.argtypes = [_P, _P, _P, _I, _I, _I, _I, _P]
        c.velox_skinny_glu_rows_bf16.restype = _I
        c.velox_skinny_gemm_splitk_bf16.argtypes = [_P, _P, _P, _I, _I, _I, _I, _I, _P]
        c.velox_skinny_gemm_splitk_bf16.restype = _I
        c.velox_argmax.argtypes = [_P, _P, _P, _I, _I, _I, _P]
        c.velox_sample.argtypes = [_P, _P, _P, _I, _I, _P]
        c.velox_count_tokens.argtypes = [_P, _P, _I, _I, _P]
        c.velox_count_sampled.argtypes = [_P, _P, _P, _I, _I, _P]
        c.velox_penalties_from_counts.argtypes = [_P, _P, _P, _P, _I, _I, _I, _P]
        c.velox_sample_chunked.argtypes = [_P, _P, _P, _I, _I, _I, _P, ctypes.c_longlong, _I, _P]
        c.velox_sample_chunked_scratch_bytes.argtypes = [_I, _I]
        c.velox_sample_chunked_scratch_bytes.restype = ctypes.c_longlong
        c.velox_apply_penalties.argtypes = [_P, _P, _P, _P, _I, _I, _I, _P]
        c.velox_probe_read.argtypes = [_P, ctypes.c_longlong, _P, _I, _P]
        c.velox_probe_read.restype = _I
        c.velox_probe_mfma.argtypes = [_I, _I, _P, _P]
        c.velox_probe_mfma.restype = _I
        c.velox_probe_grid_barrier.argtypes = [_I, _I, _I, _P, _P, _P]
        c.velox_probe_grid_barrier.restype = _I
        for fn in (c.velox_embed, c.velox_place_tokens, c.velox_add_rmsnorm, c.velox_silu_mul, c.velox_rope_kv_write, c.velox_gemm_fma,
                   c.velox_argmax, c.velox_sample, c.velox_sample_chunked, c.velox_apply_penalties, c.velox_count_tokens, c.velox_count_sampled,
                   c.velox_penalties_from_counts):
            fn.restype = _I

    def attention_library(self, head_dim: int) -> ctypes.CDLL:
        lib = self._attention.get(head_dim)
        if lib is None:
            lib = ctypes.CDLL(build.ensure_attention(head_dim))
            lib.velox_paged_attention.argtypes = [_P, _I, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _I, _P]
            lib.velox_paged_attention.restype = _I
            lib.velox_attention_head_dim.restype = _I
            lib.velox_attention_portion_kernel.argtypes = [_I]
            lib.velox_attention_portion_kernel.restype = None
            if lib.velox_attention_head_dim() != head_dim:
                raise KernelError(f"attention library for head_dim={head_dim} reports {lib.velox_attention_head_dim()}")
            self._attention[head_dim] = lib
        return lib

    def prepare(self, model, dtype) -> None:
        """Lets every part get what it needs of the kernels before the first step (``Part.prepare_kernels``): the weights
        that decode-sized products read are registered, and libraries that are built per size (attention, per head
        size) are built and loaded by the parts that use them."""
        for part in model.all_parts():
            part.prepare_kernels(self)
        if dtype == torch.bfloat16 and self.use_library_gemm and self._mm_out_dtype_ok is None:
            self._decide_float32_out_route()

    def prepare_weight(self, weight: torch.Tensor, stacked: int = 1, rotary_heads: Optional[Tuple[int, int, int]] = None,
                       handle: Optional[PreparedWeight] = None) -> Optional[PreparedWeight]:
        """A second copy of a bfloat16 ``[N, K]`` weight in the order the skinny kernels' lanes read it (see
        ``pack_rows``): decode-sized products then stream contiguous kilobytes.  ``stacked`` = 2 marks ``[Wgate; Wup]``;
        ``rotary_heads = (heads, kv_heads, head_dim)`` marks ``[Wq; Wk; Wv]`` whose product is followed by a rotation of
        whole heads and gets a further copy for ``qkv_rope_write``.  Each copy costs the weight's size again in memory;
        ``pack_decode_weights = False`` turns them off.  Returns what the caller keeps and passes in the weight's place
        (``handle``: an earlier result for the same weight, which is extended), or None when the kernels read this weight
        as it is."""
        if (not self.pack_decode_weights or weight is None or weight.dtype != torch.bfloat16 or weight.dim() != 2
                or weight.shape[1] % 64 != 0 or weight.shape[0] % stacked != 0 or weight.device != self.device):
            return handle
        if handle is None or handle.weight is not weight or handle.version != weight._version:
            handle = PreparedWeight(weight)
        copies = handle.copies
        if stacked not in copies:
            per_matrix = weight.shape[0] // stacked
            whole_tiles = [c for key, c in copies.items() if key in (1, 2)] if per_matrix % 16 == 0 else []
            # with whole tiles every stacking gives the same bytes
            copies[stacked] = whole_tiles[0] if whole_tiles else self.pack_rows(weight, stacked)
        if rotary_heads is not None and "rotary" not in copies:
            heads, kv_heads, head_dim = rotary_heads
            if head_dim % 32 == 0 and weight.shape[0] == (heads + 2 * kv_heads) * head_dim:
                copies["rotary"] = self.pack_rows(weight[self.rotary_row_order(heads, kv_heads, head_dim, weight.device)])
        return handle

    @staticmethod
    def rotary_row_order(heads: int, kv_heads: int, head_dim: int, device) -> torch.Tensor:
        """Row order of ``[Wq; Wk; Wv]`` for ``qkv_rope_write``: inside every query and key head, 16 channels of the low
        half are followed by their 16 partners of the high half; value heads keep their order."""
        half = head_dim // 2
        inside = torch.arange(half, device=device).view(half // 16, 1, 16) + torch.tensor([0, half], device=device).view(1, 2, 1)
        rotary = (torch.arange(heads + kv_heads, device=device).view(-1, 1) * head_dim + inside.reshape(1, -1)).reshape(-1)
        values = torch.arange((heads + kv_heads) * head_dim, (heads + 2 * kv_heads) * head_dim, device=device)
        return torch.cat([rotary, values])

    def library_serves(self, m: int, n: int, k: int) -> bool:
        """Whether ``linear`` hands ``x[m, k] @ w[n, k]^T`` in bfloat16 to the matrix library, and the product is large
        enough for the library's timing of its candidates to mean something (a weight of a few megabytes is timed
        from the caches, which says little about a step that streams it from memory)."""
        if not self.use_library_gemm:
            return False
        if m > 64:
            return True
        return m > 16 and n > 8192 and n * k >= (32 << 20)

    def tuning_file(self) -> Optional[str]:
        """Where timings of the matrix library's kernels are kept between runs by default: beside the built kernel
        libraries, one file per kind of GPU (the file's own header names the library versions it holds for, and
        TunableOp refuses a file made by others)."""
        directory = next((d for d in build.build_dirs() if build._writable(d)), None)
        arch = torch.cuda.get_device_properties(self.device).gcnArchName.split(":")[0]
        return os.path.join(directory, f"tunableop_{arch}.csv") if directory else None

    def tune_library_products(self, shapes, token_counts, seconds_per_shape: float = 0.2, results_file: Optional[str] = None) -> int:
        """Lets PyTorch's TunableOp time the library's candidate kernels for ``x[M, K] @ w[N, K]^T`` at the given
        ``(N, K)`` shapes and ``M`` values, and keeps its choices for later calls.  Tuning stays off afterwards, so
        other shapes keep the library's default choice and never pay for a search.  ``results_file``: what was found is
        kept there, and shapes that an earlier run has timed are not timed again.  Returns the number of products run."""
        tunable = torch.cuda.tunable
        tunable.enable(True)
        if results_file is None:
            # TunableOp writes what it finds to a file: keep that out of the working folder
            results_file = os.path.join(tempfile.gettempdir(), f"velox_amd_tunableop_{os.getuid()}_{os.getpid()}.csv")
        if tunable.get_filename() != results_file:
            tunable.set_filename(results_file)
            if os.path.isfile(results_file) and not tunable.read_file(results_file):
                # made with other versions of the libraries, or half written: start again.  Only a file of the engine's
                # own (beside its kernel libraries, or the temporary one) is removed; a caller's file is left alone and
                # what is found now goes to a new name beside it
                own = results_file == self.tuning_file() or os.path.dirname(results_file) == tempfile.gettempdir()
                if own:
                    os.remove(results_file)
                else:
                    fresh = f"{results_file}.{os.getpid()}"
                    logger.warning("the timings in %s cannot be read by this version of the matrix library; leaving it and writing to %s", results_file, fresh)
                    results_file = fresh
                    tunable.set_filename(results_file)
        tunable.set_max_tuning_duration(int(seconds_per_shape * 1000))
        tunable.tuning_enable(True)
        done = 0
        try:
            for n, k in sorted(set(shapes)):
                # (operands like the real ones: a kernel's time and its clocks depend on the bits it moves)
                weight = torch.randn((n, k), dtype=torch.float32, device=self.device).mul_(0.02).to(torch.bfloat16)
                for m in sorted(set(token_counts)):
                    x = torch.randn((m, k), dtype=torch.float32, device=self.device).to(torch.bfloat16)
                    torch.nn.functional.linear(x, weight)
                    done += 1
                del weight
            torch.cuda.synchronize(self.device)
        finally:
            tunable.tuning_enable(False)
        return done

    # -- helpers --------------------------------------------------------------------------------
    def _stream(self):
        # (the raw handle of the current stream: the same value as torch.cuda.current_stream(device).cuda_stream, without
        # building a Stream object for every kernel call, which costs more host time than the launch itself)
        if self._raw_stream is not None:
            return _P(self._raw_stream(self.device.index))
        return _P(torch.cuda.current_stream(self.device).cuda_stream)

    def _check(self, name: str, t: torch.Tensor, dtype=None, shape=None, align: int = 4) -> None:
        if not isinstance(t, torch.Tensor) or t.device != self.device:
            raise KernelError(f"{name}: expected a tensor on {self.device}, got {getattr(t, 'device', type(t))}")
        if not t.is_contiguous():
            raise KernelError(f"{name}: must be contiguous (shape {tuple(t.shape)}, strides {t.stride()})")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")
        if t.data_ptr() % align != 0:
            raise KernelError(f"{name}: address must be a multiple of {align}")

    @staticmethod
    def _launched(status: int, what: str) -> None:
        if status != 0:
            raise KernelError(f"{what}: launch failed with HIP error {status}")

    # -- embedding and norms ----------------------------------------------------------------------
    def embed(self, token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        self._check("token_ids", token_ids, torch.int32)
        self._check("table", table)
        if token_ids.dim() != 1 or table.dim() != 2:
            raise KernelError("embed: token_ids must be [T] and the table [V, H]")
        vocab, hidden = table.shape
        out = torch.empty((token_ids.shape[0], hidden), dtype=torch.float32, device=self.device)
        status = self._core.velox_embed(_ptr(token_ids), _ptr(table), _ptr(out), token_ids.shape[0], hidden, vocab, _code(table.dtype), self._stream())
        self._launched(status, "embed")
        return out

    def place_tokens(self, ids: torch.Tensor, dest: torch.Tensor, source: torch.Tensor, tokens: torch.Tensor, count: int) -> None:
        """``ids[dest[k]] = tokens[source[k]]`` for ``k < count``, all int32 on the device: token ids that the step in flight
        is still sampling, put into this step's rows without a trip to the host."""
        for name, t in (("ids", ids), ("dest", dest), ("source", source), ("tokens", tokens)):
            self._check(name, t, torch.int32)
            if t.dim() != 1:
                raise KernelError(f"place_tokens: {name} must have one dimension")
        if count < 0 or count > dest.numel() or count > source.numel():
            raise KernelError(f"place_tokens: {count} pairs do not fit dest [{dest.numel()}] and source [{source.numel()}]")
        status = self._core.velox_place_tokens(_ptr(ids), _ptr(dest), _ptr(source), _ptr(tokens), int(count), ids.numel(), tokens.numel(), self._stream())
        self._launched(status, "place_tokens")

    def _norm(self, residual, delta, rows, weight, eps, out_dtype):
        self._check("residual", residual, torch.float32)
        if residual.dim() != 2:
            raise KernelError("add_rmsnorm: residual must be [T, H]")
        tokens, hidden = residual.shape
        self._check("weight", weight, torch.float32, (hidden,))
        partials, partial_stride = 1, 0
        if delta is not None:
            if delta.dim() == 3:  # partial sums of a split product, added here
                partials, partial_stride = delta.shape[0], tokens * hidden
                self._check("delta", delta, torch.float32, (partials, tokens, hidden), align=16)
            else:
                self._check("delta", delta, None, (tokens, hidden))
        if rows is not None:
            self._check("rows", rows, torch.int32)
            count = rows.shape[0]
        else:
            count = tokens
        out = torch.empty((count, hidden), dtype=out_dtype, device=self.device)
        delta_code = _code(delta.dtype) if delta is not None else _code(out_dtype)
        status = self._core.velox_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(rows), _ptr(weight), _ptr(out), count, hidden, float(eps), delta_code, _code(out_dtype), partials, partial_stride, self._stream())
        self._launched(status, "add_rmsnorm")
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype):
        return self._norm(residual, delta, None, weight, eps, out_dtype)

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps, out_dtype):
        return self._norm(residual, delta, rows, weight, eps, out_dtype)

    # -- matrix products --------------------------------------------------------------------------
    @staticmethod
    def _scale_args(deferred: Optional[DeferredNorm]):
        """The four arguments by which a skinny product learns how to scale its result rows."""
        if deferred is None:
            return _P(0), 0, 0.0, 0.0
        return _ptr(deferred.sums), int(deferred.sums.shape[1]), 1.0 / deferred.width, float(deferred.eps)

    def _packed_rows_of(self, x: torch.Tensor, k: int) -> Optional[torch.Tensor]:
        """The copy of decode-sized activations ``x`` [M <= 16, k] in the order the skinny kernels' lanes read them, if the
        kernel that wrote ``x`` left one (it hangs on the tensor object), else None."""
        twin, version = getattr(x, "_velox_packed_rows", (None, None))
        if (twin is None or version != x._version or x.dim() != 2 or x.shape[0] > 16 or x.shape[1] != k or k % 64 != 0
                or twin.numel() != k // 64 * 1024 or twin.dtype != torch.bfloat16):
            return None
        return twin

    def _room_for_packed_rows(self, m: int, n: int) -> Optional[torch.Tensor]:
        """Room for ``[m, n]`` activations in the lanes' order, if the kernels can write and read them like that and it
        pays: the copy always has 16 rows, and what a product's activations cost is their bytes, not the pieces they come in
        (measured on MI355X, 3584 x 18944: 12 rows row-major 28.5 us, 16 rows 30.9 us, the copy 28.4 us at any number)."""
        if not 13 <= m <= 16 or n % 64 != 0 or not self.pack_decode_weights:
            return None
        return torch.empty(n // 64 * 1024, dtype=torch.bfloat16, device=self.device)

    def materialize(self, x):
        """A ``DeferredNorm`` as the plain normalised tensor (one small kernel); anything else is returned as it is."""
        if not isinstance(x, DeferredNorm):
            return x
        m, n = x.x.shape
        out = torch.empty_like(x.x)
        sums, blocks, inv_width, eps = self._scale_args(x)
        self._launched(self._core.velox_row_scale_apply(_ptr(x.x), sums, blocks, inv_width, eps, _ptr(out), m, n, self._stream()), "row_scale_apply")
        return out

    def linear(self, x, weight: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype, partials_ok: bool = False,
               residual_norm: Optional[ResidualSink] = None):
        """``x @ weight^T (+ bias)`` as ``[M, N]`` in ``out_dtype``.  With ``partials_ok`` the result may instead come back as
        float32 partial sums ``[S, M, N]`` that the consumer adds (``add_rmsnorm`` does).  With ``residual_norm`` it may
        come back as a ``DeferredNorm``: the product has then been added to ``residual_norm.residual`` and multiplied
        with the weight of ``residual_norm.norm`` (decode-sized bfloat16 products whose weight is registered).  ``x`` may
        be a ``DeferredNorm``."""
        weight, prepared = _weight_of(weight)
        packed = prepared.copy(1) if prepared is not None else None
        deferred = x if isinstance(x, DeferredNorm) else None
        if deferred is not None:
            x = deferred.x
            if not (self.use_skinny_gemm and packed is not None and x.shape[0] <= 16 and x.shape[1] % 64 == 0 and weight.dtype == torch.bfloat16):
                x, deferred = self.materialize(deferred), None
        self._check("x", x, align=16)
        self._check("weight", weight, align=16)
        if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
            raise KernelError(f"linear: x {tuple(x.shape)} and weight {tuple(weight.shape)} do not match")
        m, k = x.shape
        n = weight.shape[0]
        if bias is not None:
            self._check("bias", bias, torch.float32, (n,))
        if deferred is not None:
            return self.skinny_gemm(x, weight, bias, out_dtype, packed=packed, row_scale=deferred, x_packed=self._packed_rows_of(x, k))
        if residual_norm is not None and bias is None:
            fused = self._linear_into_residual(x, weight, residual_norm, packed=packed)
            if fused is not None:
                return fused
        if (partials_ok and bias is None and self.use_skinny_gemm and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                and 16 < m <= 64 and k % 64 == 0 and n <= 8192 and n % 4 == 0):
            return self.skinny_gemm_splitk(x, weight, packed=packed)
        skinny_rows = 16 if n > 8192 else 32  # measured on MI355X: beyond this the library's kernels stream faster
        if self.use_skinny_gemm and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and m <= skinny_rows and k % 64 == 0:
            return self.skinny_gemm(x, weight, bias, out_dtype, packed=packed, x_packed=self._packed_rows_of(x, k))
        if self.use_library_gemm and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and bias is None:
            if out_dtype == torch.bfloat16:
                return torch.nn.functional.linear(x, weight)
            if out_dtype == torch.float32:
                if self._mm_out_dtype_ok is None:
                    self._decide_float32_out_route()
                return torch.mm(x, weight.t(), out_dtype=torch.float32)
        return self.gemm_fma(x, weight, bias, out_dtype)

    def _decide_float32_out_route(self) -> None:
        """Decides once how a bfloat16 product with a float32 result and more rows than the skinny kernels take (the
        head over many wanted rows) is computed: by the library with a float32 output, if this PyTorch has that call.
        If it has not, that is an error here, at load time, and not a silent fall to the exact FMA kernel, which is some
        two hundred times slower at such sizes."""
        probe = torch.zeros((32, 64), dtype=torch.bfloat16, device=self.device)
        try:
            torch.mm(probe, probe.t(), out_dtype=torch.float32)
            self._mm_out_dtype_ok = True
        except (RuntimeError, TypeError) as err:
            self._mm_out_dtype_ok = False
            raise KernelError("this PyTorch's matrix library has no bfloat16 product with a float32 result (torch.mm(..., out_dtype=)); "
                              f"logits of many rows at once need it in a bfloat16 run: {err}") from err

    def _linear_into_residual(self, x: torch.Tensor, weight: torch.Tensor, sink: ResidualSink, waves: Optional[int] = None, row_tiles: Optional[int] = None,
                              packed: Optional[torch.Tensor] = None) -> Optional[DeferredNorm]:
        """``sink.residual += x @ weight^T`` with the first half of ``sink.norm`` in the same kernel, if this product
        qualifies (bfloat16, at most 16 rows, registered weight, a norm that can be split); None otherwise."""
        form = sink.norm.deferred_form()
        weight, prepared = _weight_of(weight)
        if prepared is not None and packed is None:
            packed = prepared.copy(1)
        m, k = x.shape
        n = weight.shape[0]
        residual = sink.residual
        if (not self.use_skinny_gemm or not self.fuse_residual_norm or form is None or packed is None or m > 16 or k % 64 != 0 or n > 16 * 512
                or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16):
            return None
        norm_weight, eps = form
        self._check("residual", residual, torch.float32, (m, n), align=16)
        self._check("norm weight", norm_weight, torch.float32, (n,))
        blocks = (n + 15) // 16
        if row_tiles is None:
            # one 16-row tile of the weight per workgroup while that is at most one workgroup per compute unit; a wider
            # weight takes two (measured on MI355X at 8 rows: 5120 x 27648 65.8 -> 58.5 us, 3584 x 18944 27.8 -> 41.4)
            # and a narrow one half a tile, which gives every compute unit a workgroup (1536 x 8960: 13.0 -> 10.8 us)
            row_tiles = 2 if blocks > self.num_cus else 0 if 2 * blocks <= self.num_cus else 1
        if row_tiles == 0:
            blocks *= 2  # (half a tile per workgroup: sums of squares per 8 columns)
        out = torch.empty((m, n), dtype=torch.bfloat16, device=self.device)
        sums = torch.empty((16, blocks), dtype=torch.float32, device=self.device)
        x_packed = self._packed_rows_of(x, k)
        out_packed = self._room_for_packed_rows(m, n)
        status = self._core.velox_skinny_residual_norm_bf16(_ptr(x if x_packed is None else x_packed), _ptr(packed), _ptr(residual), _ptr(norm_weight),
                                                            _ptr(out), _ptr(sums), m, n, k, int(waves or 8), int(row_tiles), int(x_packed is not None), _ptr(out_packed),
                                                            self._stream())
        self._launched(status, "skinny_residual_norm")
        if out_packed is not None:
            out._velox_packed_rows = (out_packed, out._version)
        return DeferredNorm(out, sums, n, float(eps), sink.norm)

    @staticmethod
    def pack_rows(weight: torch.Tensor, matrices: int = 1) -> torch.Tensor:
        """``weight`` [N, K] bfloat16 (``matrices`` stacked matrices of N / matrices rows each) in the order the skinny
        kernels' lanes read it: [row tile of 16][block of 64 indices][half h][lane = 16 * g + row][8 elements] holds index
        ``16 g + 8 h + e`` of the block; each matrix is padded with zero rows to whole tiles.  Each of a wave's two loads of
        a block is then one contiguous kilobyte."""
        n_all, k = weight.shape
        n = n_all // matrices
        tiles = (n + 15) // 16
        padded = torch.zeros((matrices, tiles * 16, k), dtype=weight.dtype, device=weight.device)
        padded[:, :n] = weight.view(matrices, n, k)
        # [matrix, tile, row i, block, group g, half h, 8] -> [matrix, tile, block, h, g, i, 8]
        return padded.view(matrices, tiles, 16, k // 64, 4, 2, 8).permute(0, 1, 3, 5, 4, 2, 6).contiguous().view(-1)

    def skinny_gemm(self, x, weight, bias, out_dtype, waves: Optional[int] = None, row_tiles: Optional[int] = None, packed: Optional[torch.Tensor] = None, n: Optional[int] = None,
                    row_scale: Optional[DeferredNorm] = None, x_packed: Optional[torch.Tensor] = None):
        """Few rows (M <= 64) times a bfloat16 weight: the weight-streaming kernel of the decode step.  ``packed`` is
        ``pack_rows(weight)``, used instead of ``weight`` when given (``n`` = rows of the weight).  ``row_scale``: ``x`` is
        its ``.x`` and the result rows are scaled as it says (M <= 16)."""
        m, k = x.shape
        n = weight.shape[0] if weight is not None else n
        if packed is not None:
            weight_arg = packed
            if packed.dtype != torch.bfloat16 or packed.numel() != ((n + 15) // 16) * 16 * k:
                raise KernelError("skinny_gemm: the packed weight does not match N and K")
        else:
            weight_arg = weight
        if x.dtype != torch.bfloat16 or weight_arg.dtype != torch.bfloat16 or m > 64 or k % 64 != 0:
            raise KernelError(f"skinny_gemm: needs bfloat16 operands, M <= 64 and K % 64 == 0 (M={m}, K={k})")
        if row_tiles is None:
            # 64 rows per wave quarter the activation traffic, which pays for the row-major weight only
            row_tiles = 4 if (m <= 16 and n >= 64 * 2 * self.num_cus and (packed is None or m > 8)) else 1
        if waves is None and packed is not None and row_tiles == 1 and m <= 16:
            waves = 8
        if waves is None:
            rows_per_block = 16 * row_tiles if m <= 16 else 32
            blocks = (n + rows_per_block - 1) // rows_per_block
            wanted = (8 * self.num_cus + blocks - 1) // blocks  # about eight waves per SIMD lane group across the GPU
            waves = 16 if wanted > 8 else 8 if wanted > 4 else 4
        out = torch.empty((m, n), dtype=out_dtype, device=self.device)
        if row_scale is not None and m > 16:
            raise KernelError("skinny_gemm: rows are scaled only for M <= 16")
        if x_packed is not None and (m > 16 or x_packed.dtype != torch.bfloat16 or x_packed.numel() != k // 64 * 1024):
            raise KernelError("skinny_gemm: the packed activations do not match M and K")
        status = self._core.velox_skinny_gemm_bf16(_ptr(x if x_packed is None else x_packed), _ptr(weight_arg), _ptr(bias), _ptr(out), m, n, k, _code(out_dtype),
                                                   int(waves), int(row_tiles), 1 if packed is not None else 0, *self._scale_args(row_scale),
                                                   int(x_packed is not None), self._stream())
        self._launched(status, "skinny_gemm")
        return out

    def linear_silu_mul(self, x: torch.Tensor, gate_up_weight: torch.Tensor, out_dtype: torch.dtype, waves: Optional[int] = None, pairs: Optional[int] = None, packed: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``silu(x Wgate^T) * (x Wup^T)`` for ``W = [Wgate; Wup]``.  Decode-sized bfloat16 batches run as one kernel that
        never writes the [M, 2I] product (up to 16 rows on any weight, 17 .. 64 rows on a registered one); everything else
        is the product followed by the SiLU kernel.  ``waves`` and ``pairs`` override the launch shape the wrapper would
        pick (up to 16 rows: waves per workgroup and gate/up tile pairs per wave; 17 .. 64 rows: ``pairs`` = tile pairs per
        workgroup)."""
        operand = gate_up_weight  # (as given: handed on to ``linear`` when nothing here applies)
        gate_up_weight, prepared = _weight_of(gate_up_weight)
        if packed is None and prepared is not None:
            packed = prepared.copy(2)
        deferred = x if isinstance(x, DeferredNorm) else None
        if deferred is not None:
            x = deferred.x
        m, k = x.shape
        two_n = gate_up_weight.shape[0]
        fused = (self.use_skinny_gemm and x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16 and out_dtype == torch.bfloat16
                 and m <= 16 and k % 64 == 0 and two_n % 2 == 0 and x.dim() == 2 and gate_up_weight.shape[1] == k)
        if (not fused and deferred is None and self.use_skinny_gemm and x.dim() == 2 and 16 < m <= 64 and k % 64 == 0 and two_n % 2 == 0
                and x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16 and out_dtype == torch.bfloat16
                and gate_up_weight.shape[1] == k and packed is not None):
            # 17 .. 64 rows: the kernel that streams the packed weight once with the activation as its epilogue
            n = two_n // 2
            if packed.dtype != torch.bfloat16 or packed.numel() != 2 * ((n + 15) // 16) * 16 * k:
                raise KernelError("linear_silu_mul: the packed weight does not match N and K")
            self._check("x", x, torch.bfloat16, align=16)
            out = torch.empty((m, n), dtype=torch.bfloat16, device=self.device)
            # pairs of tiles per workgroup: a compute unit holds one such workgroup at a time, so the launch takes
            # rounds x pairs; the fewest wins, then the larger workgroup (measured on MI355X at 64 rows: 37888 x 3584
            # with 5 pairs 51 us, the library's product + SiLU kernel 58; 55296 x 5120 with 4 pairs 106 us against 114)
            tiles = (n + 15) // 16
            per_group = min(range(2, 7), key=lambda p: (-(-(-(-tiles // p)) // self.num_cus) * p, -p))
            self._launched(self._core.velox_skinny_glu_rows_bf16(_ptr(x), _ptr(packed), _ptr(out), m, n, k, per_group if pairs is None else int(pairs), self._stream()),
                           "skinny_glu_rows")
            return out
        if not fused:
            return self.silu_mul(self.linear(deferred if deferred is not None else x, operand, None, out_dtype))
        if deferred is not None and packed is None:  # only the kernels of a registered weight scale rows
            x, deferred = self.materialize(deferred), None
        self._check("x", x, align=16)
        self._check("gate_up_weight", gate_up_weight, align=16)
        n = two_n // 2
        if pairs is None:
            pairs = 1  # measured on MI355X: two pairs per wave never paid, packed or not
        if waves is None:
            waves = 8
        out = torch.empty((m, n), dtype=out_dtype, device=self.device)
        x_packed = self._packed_rows_of(x, k)
        out_packed = self._room_for_packed_rows(m, n)
        status = self._core.velox_skinny_gemm_glu_bf16(_ptr(x if x_packed is None else x_packed), _ptr(packed if packed is not None else gate_up_weight), _ptr(out),
                                                       m, n, k, int(waves), int(pairs), 1 if packed is not None else 0, *self._scale_args(deferred),
                                                       int(x_packed is not None), _ptr(out_packed), self._stream())
        self._launched(status, "skinny_gemm_glu")
        if out_packed is not None:
            out._velox_packed_rows = (out_packed, out._version)
        return out

    def skinny_gemm_splitk(self, x, weight, splits: Optional[int] = None, packed: Optional[torch.Tensor] = None) -> torch.Tensor:
        """17 .. 64 rows times a bfloat16 weight with few rows and a long K: float32 partial sums ``[S, M, N]``.
        ``packed``: ``pack_rows(weight)``, read instead of ``weight`` when given."""
        m, k = x.shape
        n = weight.shape[0]
        if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or m > 64 or k % 64 != 0:
            raise KernelError(f"skinny_gemm_splitk: needs bfloat16 operands, M <= 64 and K % 64 == 0 (M={m}, K={k})")
        self._check("x", x, align=16)
        self._check("weight", weight, align=16)
        if splits is None:
            # one workgroup per compute unit (measured on MI355X: a unit that gets a second one holds the others up)
            blocks = (n + 63) // 64
            splits = max(1, min(self.num_cus // blocks, k // 256, 16))
        per_split = (k // 64 + splits - 1) // splits
        splits = (k // 64 + per_split - 1) // per_split  # no empty slice
        out = torch.empty((splits, m, n), dtype=torch.float32, device=self.device)
        if packed is not None and (packed.dtype != torch.bfloat16 or packed.numel() != ((n + 15) // 16) * 16 * k):
            raise KernelError("skinny_gemm_splitk: the packed weight does not match N and K")
        status = self._core.velox_skinny_gemm_splitk_bf16(_ptr(x), _ptr(weight if packed is None else packed), _ptr(out), m, n, k, splits,
                                                          int(packed is not None), self._stream())
        self._launched(status, "skinny_gemm_splitk")
        return out

    def gemm_fma(self, x, weight, bias, out_dtype):
        m, k = x.shape
        n = weight.shape[0]
        out = torch.empty((m, n), dtype=out_dtype, device=self.device)
        status = self._core.velox_gemm_fma(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, _code(x.dtype), _code(weight.dtype), _code(out_dtype), self._stream())
        self._launched(status, "gemm_fma")
        return out

    def silu_mul(self, gate_up: torch.Tensor) -> torch.Tensor:
        self._check("gate_up", gate_up)
        if gate_up.dim() != 2 or gate_up.shape[1] % 2 != 0:
            raise KernelError("silu_mul: expected [T, 2 * intermediate]")
        tokens, inter = gate_up.shape[0], gate_up.shape[1] // 2
        out = torch.empty((tokens, inter), dtype=gate_up.dtype, device=self.device)
        status = self._core.velox_silu_mul(_ptr(gate_up), _ptr(out), tokens, inter, _code(gate_up.dtype), self._stream())
        self._launched(status, "silu_mul")
        return out

    # -- rotary + cache write ---------------------------------------------------------------------
    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=True, bias=None):
        tokens = qkv.shape[0]
        width = (num_heads + 2 * num_kv_heads) * head_dim
        self._check("qkv", qkv, None, (tokens, width), align=16)
        self._check("positions", positions, torch.int32, (tokens,))
        self._check("slot_mapping", slot_mapping, torch.int32, (tokens,))
        if bias is not None:
            self._check("bias", bias, torch.float32, (width,))
        half = 0
        if cos is not None:
            self._check("cos", cos, torch.float32)
            self._check("sin", sin, torch.float32, tuple(cos.shape))
            half = cos.shape[1]
            if 2 * half > head_dim:
                raise KernelError(f"rotary span {2 * half} exceeds head_dim {head_dim}")
        pages = k_cache.shape[0]
        self._check("k_cache", k_cache, qkv.dtype, (pages, num_kv_heads, block_size, head_dim), align=16)
        self._check("v_cache", v_cache, qkv.dtype, (pages, num_kv_heads, head_dim, block_size), align=16)
        # positions index the tables and slots index the cache: both are built by the batch builder from
        # block tables the cache manager handed out, bounded by max_model_len and the pool size
        status = self._core.velox_rope_kv_write(
            _ptr(qkv), _ptr(bias), _ptr(positions), _ptr(cos), _ptr(sin), half, _ptr(slot_mapping), _ptr(k_cache), _ptr(v_cache),
            tokens, num_heads, num_kv_heads, head_dim, block_size, 1 if write_kv else 0, _code(qkv.dtype), self._stream())
        self._launched(status, "rope_kv_write")

    def rope_kv_write_partial(self, partial, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size,
                              write_kv=True, bias=None) -> torch.Tensor:
        """``rope_kv_write`` on rows that come as float32 partial sums ``[S, M, (heads + 2 kv_heads) * head_dim]`` (bfloat16
        caches): returns bfloat16 ``[M, width]`` whose query columns hold the rotated queries (the others are not written)."""
        if partial.dim() != 3:
            raise KernelError("rope_kv_write_partial: partial sums are [S, M, width]")
        parts, tokens, width = partial.shape
        if width != (num_heads + 2 * num_kv_heads) * head_dim or head_dim % 16 != 0:
            raise KernelError(f"rope_kv_write_partial: rows of {width} elements do not hold {num_heads} + 2 x {num_kv_heads} heads of {head_dim}")
        self._check("partial", partial, torch.float32, (parts, tokens, width), align=16)
        self._check("positions", positions, torch.int32, (tokens,))
        self._check("slot_mapping", slot_mapping, torch.int32, (tokens,))
        if bias is not None:
            self._check("bias", bias, torch.float32, (width,), align=16)
        half = 0
        if cos is not None:
            self._check("cos", cos, torch.float32, align=16)
            self._check("sin", sin, torch.float32, tuple(cos.shape), align=16)
            half = cos.shape[1]
            if 2 * half != head_dim:
                raise KernelError("rope_kv_write_partial: the rotation has to span the whole head")
        pages = k_cache.shape[0]
        self._check("k_cache", k_cache, torch.bfloat16, (pages, num_kv_heads, block_size, head_dim), align=16)
        self._check("v_cache", v_cache, torch.bfloat16, (pages, num_kv_heads, head_dim, block_size), align=16)
        out = torch.empty((tokens, width), dtype=torch.bfloat16, device=self.device)
        status = self._core.velox_rope_kv_write_partial_bf16(
            _ptr(out), _ptr(partial), parts, _ptr(bias), _ptr(positions), _ptr(cos), _ptr(sin), half, _ptr(slot_mapping), _ptr(k_cache), _ptr(v_cache),
            tokens, num_heads, num_kv_heads, head_dim, block_size, 1 if write_kv else 0, self._stream())
        self._launched(status, "rope_kv_write_partial")
        return out

    def qkv_rope_write(self, x, weight, bias, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache,
                       block_size, write_kv=True, waves: Optional[int] = None, fused: Optional[bool] = None) -> torch.Tensor:
        """Projects ``x`` with ``weight = [Wq; Wk; Wv]``, adds ``bias``, rotates queries and keys and writes keys and values
        into the cache.  Returns a tensor whose first ``num_heads * head_dim`` columns are the rotated queries (it may be
        wider).  Decode-sized bfloat16 batches run as one kernel when ``weight`` is what ``prepare_weight(w, rotary_heads=...)``
        returned; everything else is the product followed by ``rope_kv_write``."""
        operand = weight
        weight, prepared = _weight_of(weight)
        deferred = x if isinstance(x, DeferredNorm) else None
        if deferred is not None:
            x = deferred.x
        m, k = x.shape
        packed = prepared.copy("rotary") if prepared is not None else None
        can_fuse = (self.use_skinny_gemm and packed is not None and write_kv and x.dtype == torch.bfloat16 and m <= 16 and k % 64 == 0
                    and cos is not None and 2 * cos.shape[1] == head_dim and head_dim % 32 == 0 and k_cache.dtype == torch.bfloat16)
        if fused is None:
            fused = can_fuse
        elif fused and not can_fuse:
            raise KernelError("qkv_rope_write: this call cannot run fused")
        if not fused:
            n = weight.shape[0]
            if (deferred is None and self.use_skinny_gemm and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16
                    and 16 < m <= 64 and k % 64 == 0 and n <= 8192 and n == (num_heads + 2 * num_kv_heads) * head_dim and head_dim % 16 == 0
                    and (cos is None or 2 * cos.shape[1] == head_dim)):
                # 17 .. 64 rows: the split-K kernel streams the weight faster than the library's choice (measured on
                # MI355X: 15 us against 21 for 4608 x 3584 at 64 rows), and the rotation adds its partial sums
                partial = self.skinny_gemm_splitk(x, weight, packed=prepared.copy(1) if prepared is not None else None)
                return self.rope_kv_write_partial(partial, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache,
                                                  block_size, write_kv=write_kv, bias=bias)
            qkv = self.linear(deferred if deferred is not None else x, operand, None, x.dtype)
            self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size,
                               write_kv=write_kv, bias=bias)
            return qkv
        width = (num_heads + 2 * num_kv_heads) * head_dim
        self._check("x", x, torch.bfloat16, align=16)
        if weight.shape != (width, k):
            raise KernelError(f"qkv_rope_write: weight {tuple(weight.shape)} is not [{width}, {k}]")
        self._check("positions", positions, torch.int32, (m,))
        self._check("slot_mapping", slot_mapping, torch.int32, (m,))
        if bias is not None:
            self._check("bias", bias, torch.float32, (width,), align=16)
        self._check("cos", cos, torch.float32, align=16)
        self._check("sin", sin, torch.float32, tuple(cos.shape), align=16)
        pages = k_cache.shape[0]
        self._check("k_cache", k_cache, torch.bfloat16, (pages, num_kv_heads, block_size, head_dim), align=16)
        self._check("v_cache", v_cache, torch.bfloat16, (pages, num_kv_heads, head_dim, block_size), align=16)
        q = torch.empty((m, num_heads * head_dim), dtype=torch.bfloat16, device=self.device)
        x_packed = self._packed_rows_of(x, k)
        status = self._core.velox_skinny_qkv_rotary_bf16(
            _ptr(x if x_packed is None else x_packed), _ptr(packed), _ptr(bias), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping), _ptr(q), _ptr(k_cache),
            _ptr(v_cache), m, k, num_heads, num_kv_heads, head_dim, block_size, int(waves or 8), *self._scale_args(deferred),
            int(x_packed is not None), self._stream())
        self._launched(status, "skinny_qkv_rotary")
        return q

    # -- attention ------------------------------------------------------------------------------
    def choose_splits(self, num_seqs: int, num_kv_heads: int, row_tiles: int, max_kv_len: int, all_decode: bool) -> int:
        """Splits of the key range for an all-decode step (reference ``src/decode_attention.py:237-252``: enough
        workgroups to fill the GPU).  Measured on MI355X the streaming kernel runs best with one workgroup per compute
        unit: more of them add partial results to write and merge and gain nothing.  At least 64 keys per split."""
        if not all_decode:
            return 1
        base = num_seqs * num_kv_heads * row_tiles
        splits = max(1, min(self.num_cus // max(base, 1), 32, max_kv_len // 64))
        # Splits and their merge cost about 3 us; a workgroup streams 64 keys in about 0.7 us.  Behind few keys one
        # workgroup per sequence and KV head is quicker (measured on MI355X, one sequence of 256 keys: 7.2 us against 9.4
        # with 4 splits; 512 keys: 9.8 us against 8.0 with 8).
        if max_kv_len * (splits - 1) < 448 * splits:
            splits = 1
        return splits

    def choose_portion_splits(self, num_tokens: int, group: int, num_kv_heads: int, max_kv_len: int) -> int:
        """Splits of the key range for portions of prompts.  Few tokens behind many keys are few workgroups that each walk
        all the keys: with the keys split the step fills the GPU with the large workgroups (measured on MI355X, 512
        tokens behind 8,192 keys: 157 us in one pass, 104 us in four splits and their merge; behind 32,768: 611 and 331).
        At least 1,024 keys per split, and none below 4,096 keys, where one pass is as quick."""
        if max_kv_len < 4096:
            return 1
        blocks = max(1, num_tokens * group // 128 * num_kv_heads)  # workgroups of 128 rows, as the launch counts them
        if blocks >= self.num_cus:
            return 1
        return max(1, min(-(-self.num_cus // blocks), max_kv_len // 1024, 16))

    def attention_scratch_elems(self, num_heads: int, num_kv_heads: int, head_dim: int, max_num_tokens: int, max_num_seqs: int, max_model_len: int) -> Tuple[int, int]:
        """The most float32 elements ``paged_attention`` asks its workspace for (partial outputs, partial log-sums) in
        any step of at most ``max_num_tokens`` tokens and ``max_num_seqs`` sequences behind at most ``max_model_len`` keys,
        with the splits that ``choose_splits`` and ``choose_portion_splits`` pick.  The bound counts TOKENS, not sequences:
        the sequence on the null page that pads a step up to a timed number of rows (one more than ``max_num_seqs``) brings
        tokens within ``max_num_tokens`` like any other and is covered."""
        group = num_heads // num_kv_heads
        rows = 0  # splits x the rows the partial results are counted by
        for count in range(1, max_num_seqs + 1):  # single tokens, alone or before portions
            rows = max(rows, count * self.choose_splits(count, num_kv_heads, 1, max_model_len, True))
        for portion in range(1, max_num_tokens + 1):  # portions of prompts, behind up to max_num_seqs - 1 single tokens
            whole = min(max_num_tokens, portion + max_num_seqs - 1)
            rows = max(rows, whole * self.choose_portion_splits(portion, group, num_kv_heads, max_model_len))
        return rows * num_heads * head_dim, rows * num_heads

    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_size, block_tables, cu_q, kv_lens,
                        max_q_len, max_kv_len, scale, window, all_decode, workspace, splits: Optional[int] = None, decode_prefix: int = 0,
                        portions_max_kv_len: Optional[int] = None):
        """Attention of every token of the step over its sequence's keys in the cache.  ``decode_prefix``: how many of the
        first sequences bring exactly one token (the engine puts decoded tokens before portions of prompts).  In a mixed
        step those run through the streaming kernel with their keys split over workgroups, the others through the
        general kernel: a single token behind many keys would otherwise be one workgroup's long walk that the
        whole step waits for.  ``portions_max_kv_len``: the most keys any sequence behind that prefix holds (default: ``max_kv_len``)."""
        tokens = qkv.shape[0]
        width = qkv.shape[1] if qkv.dim() == 2 else -1  # rows may carry keys and values after the queries
        if width not in (num_heads * head_dim, (num_heads + 2 * num_kv_heads) * head_dim):
            raise KernelError(f"paged_attention: rows of {width} elements hold neither the queries nor queries, keys and values")
        self._check("qkv", qkv, None, (tokens, width), align=16)
        num_seqs = kv_lens.shape[0]
        self._check("kv_lens", kv_lens, torch.int32, (num_seqs,))
        self._check("cu_q", cu_q, torch.int32, (num_seqs + 1,))
        self._check("block_tables", block_tables, torch.int32)
        if block_tables.dim() != 2 or block_tables.shape[0] != num_seqs:
            raise KernelError(f"block_tables must be [{num_seqs}, W], got {tuple(block_tables.shape)}")
        if block_size <= 0 or block_size & (block_size - 1):
            raise KernelError(f"block_size must be a power of two, got {block_size}")
        if block_tables.shape[1] * block_size < max_kv_len:
            raise KernelError(f"block tables of width {block_tables.shape[1]} cannot cover {max_kv_len} keys")
        pages = k_cache.shape[0]
        self._check("k_cache", k_cache, qkv.dtype, (pages, num_kv_heads, block_size, head_dim), align=16)
        self._check("v_cache", v_cache, qkv.dtype, (pages, num_kv_heads, head_dim, block_size), align=16)
        if num_heads % num_kv_heads != 0:
            raise KernelError("num_heads must be a multiple of num_kv_heads")
        if not scale > 0:
            raise KernelError(f"paged_attention: the scale must be positive, got {scale}")
        if max_q_len < 1 or max_q_len > tokens:
            raise KernelError(f"max_q_len={max_q_len} outside [1, {tokens}]")
        if not 0 <= decode_prefix <= num_seqs or num_seqs > tokens:
            raise KernelError(f"decode_prefix={decode_prefix} does not fit {num_seqs} sequences with {tokens} tokens")
        lib = self.attention_library(head_dim)
        group = num_heads // num_kv_heads
        out = torch.empty((tokens, num_heads * head_dim), dtype=qkv.dtype, device=self.device)

        def launch(first_seq: int, count: int, first_token: int, num_tokens: int, longest: int, decode_only: bool, splits: Optional[int]) -> None:
            # sequences [first_seq, first_seq + count); their tokens are rows [first_token, first_token + num_tokens) of qkv
            # and out.  cu_q holds absolute rows, so the general kernel takes qkv and out whole; the streaming kernel
            # counts rows from its first sequence and takes the slices.
            row_tiles = (longest * group + 63) // 64
            if splits is None:
                splits = self.choose_splits(count, num_kv_heads, row_tiles, max_kv_len, decode_only)
                if not decode_only:
                    splits = self.choose_portion_splits(num_tokens, group, num_kv_heads, min(max_kv_len, portions_max_kv_len or max_kv_len))
            if count * splits > 65535:
                raise KernelError(f"{count} sequences x {splits} splits exceed the launch grid")
            part_o = part_lse = None
            if splits > 1:
                if workspace is None:
                    raise KernelError("split attention needs a workspace")
                span = num_tokens if decode_only else tokens  # the rows the kernels count partial results by
                part_o = workspace.get("attention_partial_out", splits * span * num_heads * head_dim)
                part_lse = workspace.get("attention_partial_lse", splits * span * num_heads)
            rows_in, rows_out = (qkv[first_token:first_token + num_tokens], out[first_token:first_token + num_tokens]) if decode_only else (qkv, out)
            status = lib.velox_paged_attention(
                _ptr(rows_in), width, _ptr(k_cache), _ptr(v_cache), _ptr(block_tables[first_seq:]), block_tables.shape[1],
                _ptr(cu_q[first_seq:]), _ptr(kv_lens[first_seq:]), _ptr(rows_out), _ptr(part_o), _ptr(part_lse), count,
                num_tokens if decode_only else tokens, longest, int(max_kv_len), num_heads, num_kv_heads,
                block_size.bit_length() - 1, float(scale), int(window or 0), splits, 0 if decode_only else first_token, _code(qkv.dtype),
                self._stream())
            self._launched(status, "paged_attention")

        if not all_decode and splits is None and 0 < decode_prefix < num_seqs and group <= 16:
            launch(0, decode_prefix, 0, decode_prefix, 1, True, None)
            launch(decode_prefix, num_seqs - decode_prefix, decode_prefix, tokens - decode_prefix, max_q_len, False, None)
        else:
            launch(0, num_seqs, 0, tokens, max_q_len, bool(all_decode), splits)
        return out

    # -- sampling -------------------------------------------------------------------------------
    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        self._check("logits", logits, torch.float32)
        rows, vocab = logits.shape
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        # few rows alone would leave most of the GPU idle: the vocabulary is cut into chunks of at least 2048 entries
        chunks = max(1, min(2 * self.num_cus // rows, vocab // 2048, 256))
        partial = torch.empty((rows, chunks, 2), dtype=torch.int32, device=self.device) if chunks > 1 else None
        self._launched(self._core.velox_argmax(_ptr(logits), _ptr(out), _ptr(partial), rows, vocab, chunks, self._stream()), "argmax")
        return out

    def sample(self, logits: torch.Tensor, options: torch.Tensor, with_filter: bool = True, chunks: Optional[int] = None) -> torch.Tensor:
        """One token per row of float32 ``logits`` by the rows' ``options`` (int32 ``[rows, 6]``: see ``sample_kernel``).
        ``with_filter=False`` promises that no row has top-k or top-p (a row that has one all the same comes back as -1 when rows are cut into chunks).  ``chunks``: into how many pieces a row is cut
        (default: one workgroup per row when the rows fill the GPU, else enough pieces to fill it); the tokens do not
        depend on it."""
        self._check("logits", logits, torch.float32)
        rows, vocab = logits.shape
        self._check("options", options, torch.int32, (rows, 6))
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        if chunks is None:
            # About one workgroup per compute unit: every workgroup of a pass works out the digit before its own from the
            # row's tables again, so more chunks than fill the GPU cost more than they save (64 rows of 152,064 on
            # MI355X: 187 us whole, 86 us in 4 chunks, 148 us in 16; 8 rows: 178 us whole, 46 us in 16 chunks).
            chunks = max(1, min(self.num_cus // rows, vocab // 8192, 32))
        if chunks > 1:
            if chunks > 1024 or rows > 65535:
                raise KernelError(f"sample: {rows} rows x {chunks} chunks exceed the launch grid")
            size = int(self._core.velox_sample_chunked_scratch_bytes(rows, chunks))
            scratch = torch.empty(size, dtype=torch.uint8, device=self.device)
            status = self._core.velox_sample_chunked(_ptr(logits), _ptr(options), _ptr(out), rows, vocab, chunks, _ptr(scratch), size,
                                                     1 if with_filter else 0, self._stream())
            self._launched(status, "sample_chunked")
            return out
        self._launched(self._core.velox_sample(_ptr(logits), _ptr(options), _ptr(out), rows, vocab, self._stream()), "sample")
        return out

    def apply_penalties(self, logits, tokens, lengths, coeffs) -> None:
        self._check("logits", logits, torch.float32)
        rows, vocab = logits.shape
        self._check("tokens", tokens, torch.int32)
        if tokens.dim() != 2 or tokens.shape[0] != rows:
            raise KernelError("apply_penalties: tokens must be [rows, width]")
        self._check("lengths", lengths, torch.int32, (rows,))
        self._check("coeffs", coeffs, torch.float32, (rows, 3))
        status = self._core.velox_apply_penalties(_ptr(logits), _ptr(tokens), _ptr(lengths), _ptr(coeffs), rows, vocab, tokens.shape[1], self._stream())
        self._launched(status, "apply_penalties")

    def count_tokens(self, counts_row: torch.Tensor, tokens: torch.Tensor) -> None:
        """``counts_row[token] += 1`` for every token of int32 ``tokens`` (ids outside the row are skipped)."""
        self._check("counts_row", counts_row, torch.int32)
        self._check("tokens", tokens, torch.int32)
        if counts_row.dim() != 1 or tokens.dim() != 1:
            raise KernelError("count_tokens: a row of counts and a list of tokens are expected")
        self._launched(self._core.velox_count_tokens(_ptr(counts_row), _ptr(tokens), tokens.numel(), counts_row.numel(), self._stream()), "count_tokens")

    def count_sampled(self, counts: torch.Tensor, row_of: torch.Tensor, tokens: torch.Tensor) -> None:
        """``counts[row_of[r], tokens[r]] += 1`` for every batch row ``r`` with ``row_of[r] >= 0``."""
        self._check("counts", counts, torch.int32)
        rows = tokens.numel()
        self._check("row_of", row_of, torch.int32, (rows,))
        self._check("tokens", tokens, torch.int32, (rows,))
        if counts.dim() != 2:
            raise KernelError("count_sampled: counts must be [table rows, vocab]")
        self._launched(self._core.velox_count_sampled(_ptr(counts), _ptr(row_of), _ptr(tokens), rows, counts.shape[1], self._stream()), "count_sampled")

    def apply_penalties_from_counts(self, logits: torch.Tensor, counts: torch.Tensor, row_of: torch.Tensor, coeffs: torch.Tensor) -> None:
        """Penalises float32 ``logits`` [rows, vocab] in place: row ``r`` by the counts of table row ``row_of[r]`` (rows with
        -1 are left alone) and ``coeffs[r] = (repetition, presence, frequency)``.  The host must keep ``row_of`` inside the table."""
        self._check("logits", logits, torch.float32)
        rows, vocab = logits.shape
        self._check("counts", counts, torch.int32)
        if counts.dim() != 2 or counts.shape[1] != vocab:
            raise KernelError(f"apply_penalties_from_counts: counts must be [table rows, {vocab}], got {tuple(counts.shape)}")
        self._check("row_of", row_of, torch.int32, (rows,))
        self._check("coeffs", coeffs, torch.float32, (rows, 3))
        chunks = max(1, min(2 * self.num_cus // rows, (vocab + 2047) // 2048))
        status = self._core.velox_penalties_from_counts(_ptr(logits), _ptr(counts), _ptr(row_of), _ptr(coeffs), rows, vocab, chunks, self._stream())
        self._launched(status, "penalties_from_counts")

    # -- probes ---------------------------------------------------------------------------------
    def _timed(self, launch, repeats: int) -> float:
        """Seconds per call of ``launch`` (the best of ``repeats`` after one untimed call)."""
        launch()
        torch.cuda.synchronize(self.device)
        best = float("inf")
        for _ in range(repeats):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            launch()
            end.record()
            end.synchronize()
            best = min(best, start.elapsed_time(end) * 1e-3)
        return best

    def probe_read_bandwidth(self, num_bytes: int = 4 << 30, repeats: int = 5) -> float:
        """GB/s at which a kernel that only reads streams ``num_bytes`` of device memory (far more than the caches hold)."""
        num_bytes -= num_bytes % 16
        data = torch.empty(num_bytes, dtype=torch.uint8, device=self.device).zero_()
        sink = torch.zeros(1, dtype=torch.int32, device=self.device)
        blocks = self.num_cus * 8
        seconds = self._timed(lambda: self._launched(self._core.velox_probe_read(_ptr(data), num_bytes, _ptr(sink), blocks, self._stream()), "probe_read"), repeats)
        return num_bytes / seconds * 1e-9

    def probe_grid_barrier(self, fenced: bool, rounds: int = 2000, repeats: int = 3) -> float:
        """Microseconds per barrier across one workgroup per compute unit inside one kernel: with relaxed agent-scope
        counters only, or (``fenced``) with the release and acquire that ordinary stores and loads around it need."""
        counters = torch.zeros(17 * 32, dtype=torch.int32, device=self.device)
        failed = torch.zeros(1, dtype=torch.int32, device=self.device)

        def launch() -> None:
            counters.zero_()
            self._launched(self._core.velox_probe_grid_barrier(self.num_cus, rounds, int(fenced), _ptr(counters), _ptr(failed), self._stream()), "probe_grid_barrier")

        seconds = self._timed(launch, repeats)
        if int(failed.item()) != 0:
            raise KernelError("probe_grid_barrier: a workgroup gave up waiting for the others")
        return seconds / rounds * 1e6

    def probe_mfma_rate(self, iterations: int = 20000, repeats: int = 5) -> float:
        """TFLOP/s of independent bfloat16 32x32x16 matrix instructions, two workgroups of four waves per compute unit."""
        sink = torch.zeros(1, dtype=torch.float32, device=self.device)
        blocks = self.num_cus * 2
        seconds = self._timed(lambda: self._launched(self._core.velox_probe_mfma(blocks, iterations, _ptr(sink), self._stream()), "probe_mfma"), repeats)
        return blocks * 4 * iterations * 4 * 32768.0 / seconds * 1e-12
