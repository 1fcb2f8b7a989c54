"""`HipOps`: the kernel surface on hand-written HIP kernels for gfx950.

The kernels live in shared libraries built from `distie_amd/csrc` and are called through
ctypes with raw device pointers on torch's current HIP stream, so they take part in
stream order and in graph capture like any other launch. torch is the allocator and the
stream/graph owner; the only library routine on this path is the matrix product for
large bfloat16 operands (the reference leaves its products to a library too).

Constructing `HipOps` without a GPU, without hipcc-built libraries, or for a head size
the kernels refuse, raises: there is no fallback.
"""

from __future__ import annotations

import ctypes
import logging
from typing import Dict, Optional

import numpy as np
import torch

from ..csrc import build
from .interface import BatchMeta, Ops

_log = logging.getLogger(__name__)

_F32, _BF16 = 0, 1
_CODES = {torch.float32: _F32, torch.bfloat16: _BF16}
_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64
_F = ctypes.c_float


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 and bfloat16 tensors, not {t.dtype}") from None


def _check(status: int, name: str) -> None:
    if status == 0:
        return
    if status < 0:
        raise KernelError(f"{name}: the kernel refuses these sizes or types")
    raise KernelError(f"{name}: launch failed with HIP error {status}")


def _written(t: torch.Tensor):
    """How often `t` has been written in place, as far as anyone can know: torch's own count (every in-place
    torch operation on the tensor or on a view of it) and the count of this module's kernels that write their
    argument (`_mark_written`)."""
    return (t._version, getattr(t, "_distie_version", 0))


def _mark_written(t: torch.Tensor) -> None:
    t._distie_version = getattr(t, "_distie_version", 0) + 1


class _NotATensorYet:
    """What `HipOps` hands out in place of a tensor. Anything asked of it that only a tensor has raises
    with the way out, instead of an AttributeError far from the cause."""

    def __getattr__(self, name):
        raise KernelError(f"{type(self).__name__} is a result of the HIP kernels that is not a tensor yet (asked for "
                          f".{name}): a part that computes on the values itself calls ops.dense(value) first")


class PartialSums(_NotATensorYet):
    """The result of a matrix product whose reduction was cut into slices: float32
    [slices, rows, columns], to be added in order by whoever reads it. `linear` returns it for
    small batches (a sum across workgroups inside the product would cost more than the product);
    `add_rmsnorm`, `silu_mul` and `rope_kv_write` add the slices while they read, every other
    operation sees the finished sum through `HipOps.dense`."""

    def __init__(self, data: torch.Tensor, dtype: torch.dtype) -> None:
        self.data = data
        self.dtype = dtype                  # the dtype the finished sum would have
        self.shape = data.shape[1:]
        self.device = data.device

    @property
    def slices(self) -> int:
        return self.data.shape[0]


class PendingNorm(_NotATensorYet):
    """rmsnorm(residual) * weight, not computed yet: for steps of few rows the product that reads it computes
    it itself, in front of its own work (`distie_decode_norm_product`); anything else sees the finished
    tensor through `HipOps.dense`. Valid as long as the residual it was made from is unchanged: a write in
    place by torch (also through a view) or by one of this module's kernels between `rmsnorm` and the use is
    found out and raises, instead of a norm of the wrong values."""

    def __init__(self, residual: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype) -> None:
        self.residual = residual
        self.weight = weight
        self.eps = float(eps)
        self.dtype = dtype
        self.shape = residual.shape
        self.device = residual.device
        self.version = _written(residual)

    def check(self) -> None:
        if _written(self.residual) != self.version:
            raise KernelError("a normed value was used after the residual stream it was made from had changed")


class PendingProduct(_NotATensorYet):
    """x W^T + bias for few rows of x, not computed yet: if the next thing that happens to it is the sum into
    the residual stream, the product adds itself to the stream in place (`distie_decode_product_residual`) and
    never exists as a tensor; anything else sees the finished tensor through `HipOps.dense`."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> None:
        self.x = x
        self.weight = weight
        self.bias = bias
        self.dtype = x.dtype
        self.shape = torch.Size((x.shape[0], weight.shape[0]))
        self.device = x.device


class HipOps(Ops):
    # Steps of up to FUSED_MAX_ROWS rows can run their products with the norm in front and the residual sum behind
    # folded in (six launches a layer instead of eight, no partial sums handed on). On the device that is no
    # gain: a kernel's time here is a chain of trips to memory, and the folded-in norm or the sum across a
    # workgroup's waves adds its trip to the product's own (measured at 8 rows, 1,536 wide: gate+up 18.7 us with
    # the norm against 13.4 + 4.2 us apart; down 13.2 against 8.3 us in 14 slices, since 96 workgroups pull
    # less than 1,344; q/k/v 9.0 against 5.5 + 4.2 us). Where the host bounds a step, two launches fewer a layer
    # count: steps that are launched kernel by kernel take this path, captured steps do not.
    FUSED_MAX_ROWS = 16
    FUSED_IN_CAPTURED_STEPS = False
    # float32 products (and products against weights kept in float32) of up to ROWS_MAX_ROWS rows stream the weights
    # through `gemv_rows` (FMAs on the vector ALU); beyond that the tiled float32 kernel
    ROWS_MAX_ROWS = 64
    # bfloat16 products by rows of x: up to SKINNY_MAX_ROWS the weights are streamed by one wave per block
    # of 16 weight rows, x straight from memory (above that, the library's tiles are faster);
    SKINNY_MAX_ROWS = 16
    # on a packed copy the one-wave kernel is the faster one only up to 8 rows: at 9 to 16 rows every wave reads all
    # 16 rows of x beside its weights, and the kernel that shares x through LDS takes over (decode step at batch 12
    # and 16: 1.5B shape 1.77 -> 1.66 and 1.95 -> 1.81 ms, 7B shape 4.34 -> 3.91 and 4.92 -> 4.14 ms; at batch 8 and
    # below the one-wave kernel is level or ahead)
    ONE_WAVE_MAX_ROWS = 8
    # with a packed copy of the weight, more rows go through the kernel that shares the x tile of a workgroup in
    # LDS, in passes over the weight: up to PACKED_MAX_ROWS in a captured step (measured in the decode step: 9 %
    # faster than the library at 72 rows, 5 % at 96, 4 % slower at 128), and up to PACKED_MAX_ROWS_EAGER in a step
    # that is launched kernel by kernel, which the host bounds at these sizes: the library's products cost it
    # 18 us each and the activation and rotation kernels beside them more launches (a portion of n tokens behind
    # 512, this way and through the library, 1.5B shape: 100: 2.8 and 3.4 ms, 160: 3.1 and 3.4, 200: 3.6 and 3.5,
    # 224: 3.7 and 3.5).
    # A weight of more than PACKED_LARGE_ELEMENTS (64 MB) is not held by the memory-side cache from one pass to the
    # next: a pass takes up to 96 rows, and every further one reads the weight from memory again, which the library
    # does once. Which is faster then goes by the weight's shape (7B shape at 128 rows, the packed kernels in two
    # passes and the library's best kernel by timing, with the same flush of the caches before each: gate+up
    # [37888, 3584] 144 and 115 us, the head [152064, 3584] 535 and 297, down [3584, 18944] 75 and 91):
    #  * K longer than the weight has rows (down): the packed kernels, whose K is cut into slices, up to
    #    PACKED_MAX_ROWS_LARGE rows, captured or not;
    #  * more rows than K (gate+up, the head, a large q/k/v): one pass, PACKED_MAX_ROWS_LARGE_WIDE rows. Once the
    #    library's kernels were timed for a class of row counts (`library_timed_rows`, set by the engine's start with
    #    `tune_products`), the library takes over from 65 rows on (PACKED_MAX_ROWS_LARGE_WIDE_TIMED): untimed, its
    #    choice is good at one row count and poor at the next. 7B shape, decode step at batch 72, 80, 96, 112, 128,
    #    160, 192: 6.4, 6.6, 7.3, 8.1, 8.4, 10.4, 10.9 ms timed; 6.6, 6.8, 8.0, 8.6, 9.6, 11.7, 12.0 untimed; and with
    #    every large weight on the packed kernels up to 192 rows 6.6, 6.8, 8.0, 9.2, 9.7, 11.9, 13.3. At 24 to 64 rows
    #    the timed library is 1-3 % ahead as well (gate+up rounded to bfloat16 before the activation): left as it is.
    # The 1.5B shape's weights are small, its head large: its captured step is the same either way.
    PACKED_MAX_ROWS = 96
    PACKED_MAX_ROWS_LARGE = 192
    PACKED_MAX_ROWS_LARGE_WIDE = 96
    PACKED_MAX_ROWS_LARGE_WIDE_TIMED = 64
    PACKED_MAX_ROWS_EAGER = 192
    PACKED_LARGE_ELEMENTS = 32 << 20
    # or, for a weight of at most this many elements (too few row blocks to occupy the chip that way),
    # through the one-wave kernel once per 16 rows of x
    ROW_GROUPS_MAX_ELEMENTS = 4 << 20
    # the q/k/v product with rotation and cache write in its epilogue exists per 16 rows only; from so many rows on a
    # weight above that size runs on the wide kernel instead, with rotation and cache write as the kernel behind it
    # (7B shape, decode step: 1.5 % slower at 24 rows, the same at 32 and 48, 2.7 % faster at 64)
    WIDE_QKV_MIN_ROWS = 49
    # ... and that kernel takes more than 32 rows in two passes of 32 over a weight of at most this many elements
    # (64 MB: the second pass reads it from the memory-side cache; much larger ones would come from memory twice)
    TWO_PASS_MAX_ELEMENTS = 32 << 20
    # ... and a larger one is read once per pass: as few passes as the kernel's 96 rows a pass allow, of equal size
    # (7B shape: decode step at batch 80 6.8 ms in one pass of 80 rows, 7.7 as 64 + 16; at batch 96 8.1 and 8.3;
    # a portion of 160 tokens 7.4 ms in two passes of 80 and 8.4 in three of 64, 64 and 32)
    WIDE_PASS_MAX_BLOCKS = 6
    # attention over a portion of a prompt: from so many visible keys on, the walk over the keys is cut into so
    # many parts that run side by side (measured at 12 heads of 128, 2,048 new tokens: 3 parts are best up to
    # 4,096 keys, 5 at 8,192, 8 from 16,384 on; the kernel takes up to 16)
    PREFILL_PARTS = ((1024, 3), (8192, 5), (16384, 8))
    PREFILL_WORKGROUPS = 512         # as many workgroups a short portion's attention should have, if its keys allow
    PACKED_KEEPS_FREE = 0.3          # share of the device's memory that packed weight copies leave free
    PREFILL_F32_MIN_TOKENS = 32      # float32 steps with a portion of at least this many tokens go to the tiled float32 kernel
    # decode attention cuts the keys into runs so that about DECODE_WAVES waves are at work, with at most
    # DECODE_MAX_RUNS places for partial results per request and head. The kernel keeps two waves a SIMD (2,048 on
    # the chip); 1,536 is what the step likes best (1.5B shape, batch 32 and 64: 2.07 and 2.77 ms with 1,024, 2.02
    # and 2.71 with 1,536, 2.11 and 2.75 with 2,048; 7B shape, batch 160: 10.85, 10.05, 10.15 ms; batch 1 to 16 the same)
    DECODE_WAVES = 1536
    # where the same number of runs for every request leaves more than a fifth of those waves unused (1,024 pairs
    # of a request and a kv head: one run each), the requests of a decode step share one run length instead: the
    # shortest with which their runs together stay within DECODE_WAVES, so that a long request gets more runs than a
    # short one (256 requests on 4 kv heads, contexts of 1,050 to 3,150 keys: 263 -> 245 us a layer; contexts of one
    # length are cut as before). Everywhere else it is level or behind (32 requests: 30 -> 33 us).
    DECODE_SHARED_BELOW = 0.8
    DECODE_MAX_RUNS = 256

    def __init__(self, device="cuda:0", packed_weights=True) -> None:
        """`packed_weights` (True, False, or the roles that get one, as the parts name them in
        `prepare_linear`: "qkv", "attn_out", "gate_up", "down", "head"): keep a second copy of every bfloat16 weight in the order in which the
        matrix cores take it, for products with at most `PACKED_MAX_ROWS_EAGER` rows (decode, short portions). It doubles
        the memory of the weights and makes those products 15-25 % faster, and it is what the fused
        epilogues (activation, rotation and cache write) work on; without it products of up to
        `SKINNY_MAX_ROWS` rows stream the weights as they are stored and larger ones go to the library."""
        self.device = torch.device(device)
        if isinstance(packed_weights, (bool, int)) or packed_weights is None:
            self.packed_weights = bool(packed_weights)
            self.packed_roles = None
        else:
            self.packed_roles = frozenset(packed_weights)
            self.packed_weights = bool(self.packed_roles)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError("HipOps needs an AMD GPU (torch.cuda is not available): there is no CPU path")
        name = torch.cuda.get_device_properties(self.device).gcnArchName
        if not name.startswith("gfx950"):
            raise KernelError(f"the kernels are built for gfx950 (MI355X); this device is {name}")
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self._compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        self._lib = None
        self._tuning = False
        self.library_timed_rows = 0
        self._packed_left_out = 0
        self._ops = ctypes.CDLL(str(build.ensure("ops")))
        self._declare()
        self._attn: Dict[int, ctypes.CDLL] = {}
        # pinned staging buffers for `upload`, used in turn: [host tensor, its numpy view, event of the last copy]
        self._uploads = [[None, None, None] for _ in range(self.UPLOAD_BUFFERS)]
        self._next_upload = 0

    # ------------------------------------------------------------ plumbing
    UPLOAD_BUFFERS = 8

    def upload(self, values: np.ndarray) -> torch.Tensor:
        """Through pinned memory, so that the copy is queued like a kernel: `torch.tensor(..., device=...)` copies
        from pageable memory and returns only when everything queued before it is done, which made the host
        wait for the running step three times per sampled step."""
        values = np.ascontiguousarray(values)
        dtype = torch.from_numpy(np.empty(0, dtype=values.dtype)).dtype
        nbytes = values.nbytes
        if nbytes == 0:
            return torch.empty(values.shape, dtype=dtype, device=self.device)
        slot = self._uploads[self._next_upload]
        self._next_upload = (self._next_upload + 1) % len(self._uploads)
        if slot[2] is not None:
            slot[2].synchronize()                       # the copy made out of this buffer some calls ago is done
        if slot[0] is None or slot[0].numel() < nbytes:
            slot[0] = torch.empty(max(4096, 2 * nbytes), dtype=torch.uint8, pin_memory=True)
            slot[1] = slot[0].numpy()
            slot[2] = torch.cuda.Event()
        slot[1][:nbytes] = values.reshape(-1).view(np.uint8)
        dev = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        dev.copy_(slot[0][:nbytes], non_blocking=True)
        slot[2].record()
        return dev.view(dtype).view(values.shape)

    def _declare(self) -> None:
        o = self._ops
        o.distie_scatter_i32.argtypes = [_P, _P, _P, _I, _L, _P]
        o.distie_embed.argtypes = [_P, _P, _I, _P, _I, _I, _I, _P]
        o.distie_rmsnorm.argtypes = [_P, _P, _I, _I, _P, _I, _P, _I, _I, _I, _F, _P]
        o.distie_rope_kv_write.argtypes = [_P, _I, _I, _P, _I, _P, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _P]
        o.distie_rope_table.argtypes = [_P, _P, _P, _I, _I, _P]
        o.distie_silu_mul.argtypes = [_P, _I, _I, _P, _I, _I, _I, _P]
        o.distie_sum_slices.argtypes = [_P, _I, _L, _P, _I, _P]
        o.distie_gather_rows.argtypes = [_P, _P, _P, _I, _L, _I, _P]
        o.distie_gemm_generic.argtypes = [_P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _P]
        o.distie_gemv_rows.argtypes = [_P, _I, _P, _I, _P, _P, _I, _I, _I, _I, _P]
        o.distie_gemm_skinny_slices.argtypes = [_I, _I, _I]
        o.distie_gemm_skinny_bf16.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _P]
        o.distie_pack_rows.argtypes = [_P, _P, _P, _I, _I, _P]
        o.distie_gemm_packed_bf16.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _P]
        o.distie_gemm_packed_wide_bf16.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]
        o.distie_gemm_packed_wide_slices.argtypes = [_I, _I]
        o.distie_gemm_packed_wide_qkv_bf16.argtypes = [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]
        o.distie_gemm_packed_rotary_bf16.argtypes = [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]
        o.distie_decode_norm_fits.argtypes = [_I]
        o.distie_decode_product_residual.argtypes = [_P, _P, _P, _P, _I, _I, _I, _P]
        o.distie_decode_norm_product.argtypes = [_P, _P, _F, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P,
                                                 _I, _I, _I, _I, _I, _P]
        o.distie_argmax.argtypes = [_P, _P, _I, _I, _P, _P, _P]
        o.distie_argmax_parts.argtypes = [_I, _I]
        o.distie_sample.argtypes = [_P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _P]

    def tune_library_products(self, on: bool) -> None:
        """While on, every new shape of a large product has the library's candidate kernels timed, and the
        fastest is kept for that shape, and for the other row counts of its class of 32 rows, from then on; shapes
        first met while off take their class's choice, or the library's first. Products of up to `PACKED_MAX_ROWS`
        rows do not go to the library at all (`PACKED_MAX_ROWS_EAGER` outside captured steps; large weights:
        see there). The caller that has had every class up to some number of rows timed says so in
        `library_timed_rows`: up to there large weights with more rows than K leave the packed kernels at 65 rows."""
        self._tuning = bool(on)

    def graphs_supported(self) -> bool:
        """Every kernel launches on torch's current stream and keeps its scratch at fixed
        addresses, so a step can be captured into a HIP graph."""
        return True

    def _stream(self):
        # torch's current stream as a raw handle; the direct getter saves the 4 us a call that building a
        # Stream object costs (a step makes some 200 calls)
        if _raw_stream is not None:
            return _raw_stream(self._device_index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def attention_library(self, head_dim: int) -> ctypes.CDLL:
        lib = self._attn.get(head_dim)
        if lib is None:
            if head_dim % 2 or not 2 <= head_dim <= 256:
                raise KernelError(f"attention kernels take even head sizes up to 256, not {head_dim}")
            lib = ctypes.CDLL(str(build.ensure(f"attn_d{head_dim}")))
            lib.distie_attention_generic.argtypes = [_P, _I, _L, _P, _P, _I, _P, _P, _P, _I, _P, _P,
                                                     _I, _I, _I, _I, _F, _I, _P, _F, _P]
            lib.distie_attention_prefill_bf16.argtypes = [_P, _L, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I,
                                                          _F, _I, _I, _P, _P, _P, _I, _P]
            lib.distie_attention_prefill_f32.argtypes = lib.distie_attention_prefill_bf16.argtypes
            lib.distie_attention_decode_bf16.argtypes = [_P, _L, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I,
                                                         _I, _F, _I, _I, _I, _I, _P, _P]
            lib.distie_attention_decode_run_len.argtypes = [_P, _I, _I, _I, _P, _P]
            if lib.distie_attention_head_dim() != head_dim:
                raise KernelError("attention library was built for another head size")
            self._attn[head_dim] = lib
        return lib

    def _own(self, *tensors) -> None:
        for t in tensors:
            if t is None:
                continue
            if t.device != self.device:
                raise KernelError(f"tensor on {t.device}, kernels run on {self.device}")
            if not t.is_contiguous():
                raise KernelError("kernels take contiguous tensors")

    @staticmethod
    def _check_cache(k_cache, v_cache, kv_heads, block_size, head_dim) -> None:
        if tuple(k_cache.shape[1:]) != (kv_heads, block_size, head_dim) or \
                tuple(v_cache.shape[1:]) != (kv_heads, head_dim, block_size) or k_cache.shape[0] != v_cache.shape[0]:
            raise KernelError("cache is not k [pages, kv_heads, block_size, head_dim], "
                              "v [pages, kv_heads, head_dim, block_size]")

    # ------------------------------------------------------------ operations
    def scatter_int32(self, table, index, value):
        self._own(table, index, value)
        if table.dtype != torch.int32 or index.dtype != torch.int32 or value.dtype != torch.int32 or \
                index.shape != value.shape:
            raise KernelError("scatter_int32 takes int32 tensors, one value for each index")
        _check(self._ops.distie_scatter_i32(table.data_ptr(), index.data_ptr(), value.data_ptr(), index.numel(),
                                            table.numel(), self._stream()), "scatter_i32")
        _mark_written(table)

    def embed(self, ids, table):
        self._own(ids, table)
        out = torch.empty((ids.shape[0], table.shape[1]), dtype=torch.float32, device=self.device)
        _check(self._ops.distie_embed(ids.data_ptr(), table.data_ptr(), _code(table), out.data_ptr(),
                                      ids.shape[0], table.shape[1], table.shape[0], self._stream()), "embed")
        return out

    def _norm_later(self, residual, weight, out_dtype) -> bool:
        """The norm of these rows can be left to the product that reads it."""
        return (self.packed_weights and self._fused(residual.shape[0]) and out_dtype == torch.bfloat16 and
                residual.dtype == torch.float32 and residual.dim() == 2 and
                weight.dtype in _CODES and bool(self._ops.distie_decode_norm_fits(residual.shape[1])))

    def _fused(self, rows: int) -> bool:
        return rows <= self.FUSED_MAX_ROWS and (self.FUSED_IN_CAPTURED_STEPS or not self.captured)

    def rmsnorm(self, x, weight, eps, out_dtype):
        self._own(x, weight)
        if x.dtype != torch.float32:
            raise KernelError("rmsnorm reads the float32 residual stream")
        if self._norm_later(x, weight, out_dtype):
            return PendingNorm(x, weight, eps, out_dtype)
        return self._rmsnorm_now(x, weight, eps, out_dtype)

    def _rmsnorm_now(self, x, weight, eps, out_dtype):
        out = torch.empty(x.shape, dtype=out_dtype, device=self.device)
        _check(self._ops.distie_rmsnorm(x.data_ptr(), None, _F32, 1, weight.data_ptr(), _code(weight),
                                        out.data_ptr(), _CODES[out_dtype], x.shape[0], x.shape[1], eps,
                                        self._stream()), "rmsnorm")
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype):
        if isinstance(delta, PendingProduct):
            self._own(residual, weight)
            if residual.dtype != torch.float32 or residual.shape != delta.shape:
                raise KernelError("add_rmsnorm: residual must be float32 and shaped like delta")
            # the product adds itself to the stream; what is left is the norm of the stream
            self._product_into_residual(delta, residual)
            return self.rmsnorm(residual, weight, eps, out_dtype)
        slices = 1
        delta = self.dense(delta) if isinstance(delta, PendingNorm) else delta
        if isinstance(delta, PartialSums):
            slices, delta = delta.slices, delta.data
        self._own(residual, delta, weight)
        if residual.dtype != torch.float32 or residual.shape != delta.shape[-2:]:
            raise KernelError("add_rmsnorm: residual must be float32 and shaped like delta")
        out = torch.empty(residual.shape, dtype=out_dtype, device=self.device)
        _check(self._ops.distie_rmsnorm(residual.data_ptr(), delta.data_ptr(), _code(delta), slices,
                                        weight.data_ptr(), _code(weight), out.data_ptr(), _CODES[out_dtype],
                                        residual.shape[0], residual.shape[1], eps, self._stream()), "add_rmsnorm")
        _mark_written(residual)
        return out

    def _product_into_residual(self, product: PendingProduct, residual: torch.Tensor) -> None:
        x, weight, bias = product.x, product.weight, product.bias
        packed = getattr(weight, "_distie_packed")
        M, K = x.shape
        N = weight.shape[0]
        if packed.numel() != self._packed_elements(N, K, False):
            raise KernelError("linear: the packed copy does not belong to this weight")
        _check(self._ops.distie_decode_product_residual(
            x.data_ptr(), packed.data_ptr(), bias.data_ptr() if bias is not None else None, residual.data_ptr(),
            M, N, K, self._stream()), "decode_product_residual")
        _mark_written(residual)

    def dense(self, x):
        """The finished tensor of a value that an operation here returned in a form of its own (partial sums,
        a norm or a product that was left for later); any other tensor as it is."""
        if isinstance(x, PendingNorm):
            x.check()
            return self._rmsnorm_now(x.residual, x.weight, x.eps, x.dtype)
        if isinstance(x, PendingProduct):
            return self._linear(x.x, x.weight, x.bias, x.dtype, lazy=False)
        if not isinstance(x, PartialSums):
            return x
        out = torch.empty(tuple(x.shape), dtype=x.dtype, device=self.device)
        _check(self._ops.distie_sum_slices(x.data.data_ptr(), x.slices, out.numel(), out.data_ptr(),
                                           _CODES[x.dtype], self._stream()), "sum_slices")
        return out

    # ---- packed copies of weights: tiles of 16 rows x 32 k in the matrix cores' lane order
    @staticmethod
    def _row_map(N, gated, rotary):
        """Which row of the weight sits at each place of the packed copy's row blocks (-1: zeros)."""
        if gated:
            inter = N // 2
            j = torch.arange(-(-inter // 8) * 8, dtype=torch.int64).view(-1, 8)
            gate = torch.where(j < inter, j, -1)
            up = torch.where(j < inter, j + inter, -1)
            return torch.cat([gate, up], dim=1).reshape(-1)
        if rotary is not None:
            heads, kv_heads, dim = rotary
            lo = torch.arange(dim // 2, dtype=torch.int64).view(-1, 8)                 # [dim/16, 8]
            one = torch.cat([lo, lo + dim // 2], dim=1).reshape(-1)                   # rows of a q or k head
            turned = (torch.arange(heads + kv_heads, dtype=torch.int64)[:, None] * dim + one[None, :]).reshape(-1)
            return torch.cat([turned, torch.arange((heads + kv_heads) * dim, N, dtype=torch.int64)])
        rows = torch.full((-(-N // 16) * 16,), -1, dtype=torch.int64)
        rows[:N] = torch.arange(N)
        return rows

    @staticmethod
    def _packed_elements(N, K, gated):
        row_blocks = -(-(N // 2) // 8) if gated else -(-N // 16)
        return row_blocks * -(-K // 32) * 512

    def prepare_linear(self, weight, gated=False, rotary=None, role=None):
        if self.packed_roles is not None and role not in self.packed_roles:
            return
        if not self.packed_weights or weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] % 8:
            return
        N, K = weight.shape
        name = "_distie_packed"
        if gated:
            if N % 2:
                return
            name = "_distie_gated"
        elif rotary is not None:
            heads, kv_heads, dim = rotary
            if dim % 16 or N != (heads + 2 * kv_heads) * dim:
                rotary = None                 # the fused kernel does not take it: the plain copy serves
            else:
                name = "_distie_rotary"
        if hasattr(weight, name):
            return
        self._own(weight)
        row_map = self._row_map(N, gated, rotary)
        if row_map.numel() % 16 or int(row_map.max()) >= N or int(row_map.min()) < -1 or \
                row_map.numel() // 16 * -(-K // 32) * 512 != self._packed_elements(N, K, gated):
            raise KernelError("prepare_linear: bad row map")
        # The copies are for speed, the cache is needed: a copy that would leave less than PACKED_KEEPS_FREE of the
        # card's memory free is left out (the product then streams the stored layout), said once.
        free, total = torch.cuda.mem_get_info(self.device)
        if free - 2 * self._packed_elements(N, K, gated) < self.PACKED_KEEPS_FREE * total:
            if not self._packed_left_out:
                _log.warning("packed weight copies are left out from here on: less than %.0f %% of the device's "
                             "memory would stay free", 100 * self.PACKED_KEEPS_FREE)
            self._packed_left_out += 1
            return
        row_map = row_map.to(device=self.device, dtype=torch.int32)
        packed = torch.empty(self._packed_elements(N, K, gated), dtype=torch.bfloat16, device=self.device)
        _check(self._ops.distie_pack_rows(weight.data_ptr(), packed.data_ptr(), row_map.data_ptr(),
                                          row_map.numel() // 16, K, self._stream()), "pack_rows")
        torch.cuda.current_stream(self.device).synchronize()      # row_map is freed on return
        # the copy lives and dies with the weight
        setattr(weight, name, (packed, tuple(rotary)) if name == "_distie_rotary" else packed)

    def _norm_product(self, x: PendingNorm, packed, bias, out, mode, N, rotary=None):
        """`out` = the product of rmsnorm(x.residual) with the weight whose packed copy is `packed`, the norm
        computed inside the product."""
        x.check()
        M, K = x.shape
        table = slots = k_cache = v_cache = None
        heads = kv_heads = dim = block_size = write = 0
        if rotary is not None:
            table, slots, k_cache, v_cache, heads, kv_heads, dim, block_size, write = rotary
        ptr = lambda t: t.data_ptr() if t is not None else None
        norm_weight = x.weight
        if norm_weight.dtype != torch.float32:
            # the kernel takes the norm's weights in float32 (a bfloat16 value is one exactly); kept on the tensor
            norm_weight = getattr(x.weight, "_distie_f32", None)
            if norm_weight is None:
                norm_weight = x.weight._distie_f32 = x.weight.float()
        _check(self._ops.distie_decode_norm_product(
            x.residual.data_ptr(), norm_weight.data_ptr(), x.eps, packed.data_ptr(), ptr(bias),
            out.data_ptr(), mode, M, N, K, ptr(table), ptr(slots), ptr(k_cache), ptr(v_cache), heads, kv_heads, dim,
            block_size, write, self._stream()), "decode_norm_product")
        return out

    def linear_silu_mul(self, x, gate_up_weight):
        packed = getattr(gate_up_weight, "_distie_gated", None)
        if isinstance(x, PendingNorm) and packed is not None and gate_up_weight.shape[1] == x.shape[1]:
            N, K = gate_up_weight.shape
            if packed.numel() != self._packed_elements(N, K, True):
                raise KernelError("linear_silu_mul: the packed copy does not belong to this weight")
            out = torch.empty((x.shape[0], N // 2), dtype=torch.bfloat16, device=self.device)
            return self._norm_product(x, packed, None, out, 1, N)
        x = self.dense(x)
        if packed is None or x.dtype != torch.bfloat16 or x.shape[0] > self._packed_rows(x.shape[0], *gate_up_weight.shape):
            return self.silu_mul(self.linear(x, gate_up_weight))
        self._own(x)
        M, K = x.shape
        N = gate_up_weight.shape[0]
        if gate_up_weight.shape[1] != K:
            raise KernelError(f"linear: x is [{M}, {K}], weight is {list(gate_up_weight.shape)}")
        if packed.numel() != self._packed_elements(N, K, True):
            raise KernelError("linear_silu_mul: the packed copy does not belong to this weight")
        out = torch.empty((M, N // 2), dtype=x.dtype, device=self.device)
        if M <= self.ONE_WAVE_MAX_ROWS:
            _check(self._ops.distie_gemm_packed_bf16(x.data_ptr(), packed.data_ptr(), None, out.data_ptr(), _code(out),
                                                     M, N, K, 1, self._stream()), "gemm_packed_bf16")
        else:
            _check(self._ops.distie_gemm_packed_wide_bf16(
                x.data_ptr(), packed.data_ptr(), None, out.data_ptr(), _code(out), M, N, K, 1,
                self._pass_blocks(M, N * K), self._stream()), "gemm_packed_wide_bf16")
        return out

    def linear_rope_kv_write(self, x, weight, bias, meta, group, k_cache, v_cache, inv_freq, num_heads, num_kv_heads,
                             head_dim, write):
        held = getattr(weight, "_distie_rotary", None)
        if isinstance(x, PendingNorm) and held is not None and held[1] == (num_heads, num_kv_heads, head_dim) and \
                inv_freq is not None and 2 * inv_freq.shape[0] == head_dim and k_cache.dtype == torch.bfloat16 and \
                weight.shape[1] == x.shape[1]:
            packed = held[0]
            slots = meta.groups[group].slots
            self._own(bias, k_cache, v_cache, inv_freq, slots)
            M, K = x.shape
            N = weight.shape[0]
            if N != (num_heads + 2 * num_kv_heads) * head_dim:
                raise KernelError(f"linear: weight is {list(weight.shape)} for {num_heads} + 2 x {num_kv_heads} heads")
            if bias is not None and (bias.dtype != torch.float32 or bias.shape[0] != N):
                raise KernelError("linear: bias must be float32 [N]")
            if packed.numel() != self._packed_elements(N, K, False):
                raise KernelError("linear_rope_kv_write: the packed copy does not belong to this weight")
            self._check_cache(k_cache, v_cache, num_kv_heads, meta.block_size, head_dim)
            if M != meta.num_tokens or slots.shape[0] != M:
                raise KernelError("linear_rope_kv_write: rows do not match the batch")
            table = self._rope_table(meta, inv_freq)
            out = torch.empty((M, N), dtype=torch.bfloat16, device=self.device)
            return self._norm_product(x, packed, bias, out, 2, N, rotary=(
                table, slots, k_cache, v_cache, num_heads, num_kv_heads, head_dim, meta.block_size, 1 if write else 0))
        x = self.dense(x)
        fused = held is not None and held[1] == (num_heads, num_kv_heads, head_dim) and \
            x.dtype == torch.bfloat16 and x.shape[0] <= self._packed_rows(x.shape[0], *weight.shape) and \
            inv_freq is not None and 2 * inv_freq.shape[0] == head_dim and k_cache.dtype == torch.bfloat16
        if not fused:
            return self.rope_kv_write(self.linear(x, weight, bias), meta, group, k_cache, v_cache, inv_freq,
                                      num_heads, num_kv_heads, head_dim, write)
        packed = held[0]
        slots = meta.groups[group].slots
        self._own(x, bias, k_cache, v_cache, inv_freq, slots)
        M, K = x.shape
        N = weight.shape[0]
        if weight.shape[1] != K or N != (num_heads + 2 * num_kv_heads) * head_dim:
            raise KernelError(f"linear: x is [{M}, {K}], weight is {list(weight.shape)}")
        if bias is not None and (bias.dtype != torch.float32 or bias.shape[0] != N):
            raise KernelError("linear: bias must be float32 [N]")
        if packed.numel() != self._packed_elements(N, K, False):
            raise KernelError("linear_rope_kv_write: the packed copy does not belong to this weight")
        self._check_cache(k_cache, v_cache, num_kv_heads, meta.block_size, head_dim)
        if M != meta.num_tokens or slots.shape[0] != M:
            raise KernelError("linear_rope_kv_write: rows do not match the batch")
        if M >= self.WIDE_QKV_MIN_ROWS and N * K > self.ROW_GROUPS_MAX_ELEMENTS:
            # more than one group of 16 rows against a weight that fills the chip through the wide kernel: the
            # epilogue kernel would read the weight once per group, so the product runs wide (weights once, K in
            # slices) and the rotation with the cache write behind it adds the slices
            slices = self._ops.distie_gemm_packed_wide_slices(N, K)
            shape, dtype = ((M, N), torch.bfloat16) if slices == 1 else ((slices, M, N), torch.float32)
            product = torch.empty(shape, dtype=dtype, device=self.device)
            _check(self._ops.distie_gemm_packed_wide_qkv_bf16(
                x.data_ptr(), packed.data_ptr(), bias.data_ptr() if bias is not None else None, product.data_ptr(),
                _code(product), M, K, num_heads, num_kv_heads, head_dim, self._pass_blocks(M, N * K), self._stream()),
                "gemm_packed_wide_qkv_bf16")
            if slices > 1:
                product = PartialSums(product, torch.bfloat16)
            return self.rope_kv_write(product, meta, group, k_cache, v_cache, inv_freq, num_heads, num_kv_heads,
                                      head_dim, write)
        table = self._rope_table(meta, inv_freq)
        out = torch.empty((M, N), dtype=torch.bfloat16, device=self.device)
        _check(self._ops.distie_gemm_packed_rotary_bf16(
            x.data_ptr(), packed.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
            table.data_ptr(), slots.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), M, K, num_heads,
            num_kv_heads, head_dim, meta.block_size, 1 if write else 0, self._stream()), "gemm_packed_rotary_bf16")
        return out

    def _packed_rows(self, M: int, N: int, K: int) -> int:
        """Most rows of x that go through the kernels on the packed copy of an [N, K] weight, for a product of M rows."""
        if N * K > self.PACKED_LARGE_ELEMENTS:
            if K > N:
                return self.PACKED_MAX_ROWS_LARGE
            return self.PACKED_MAX_ROWS_LARGE_WIDE_TIMED if M <= self.library_timed_rows else self.PACKED_MAX_ROWS_LARGE_WIDE
        return self.PACKED_MAX_ROWS if self.captured else self.PACKED_MAX_ROWS_EAGER

    def _library(self):
        """The vendor library's products, called directly; loaded at the first large product."""
        if self._lib is None:
            lib = ctypes.CDLL(str(build.ensure("library")))
            lib.distie_lib_init.argtypes = [ctypes.c_int]
            lib.distie_lib_init.restype = ctypes.c_int
            lib.distie_lib_linear.argtypes = [_P, _P, _P, _P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_int64, ctypes.c_int, _P]
            lib.distie_lib_linear.restype = ctypes.c_int
            lib.distie_lib_counts.argtypes = [ctypes.POINTER(ctypes.c_long), ctypes.POINTER(ctypes.c_long)]
            lib.distie_lib_counts.restype = None
            lib.distie_lib_more_counts.argtypes = [ctypes.POINTER(ctypes.c_long)] * 3
            lib.distie_lib_more_counts.restype = None
            with torch.cuda.device(self.device):
                _check(lib.distie_lib_init(self._device_index), "lib_init")
            self._lib = lib
        return self._lib

    def library_plans(self):
        """(shapes the library has a plan for, shapes whose kernel was chosen by timing)"""
        made, timed = ctypes.c_long(0), ctypes.c_long(0)
        self._library().distie_lib_counts(ctypes.byref(made), ctypes.byref(timed))
        return made.value, timed.value

    def library_counts(self) -> dict:
        """`held`: shapes the library holds a plan for now; `asked`: how often it was asked to rank its kernels
        (row counts of one class of 32 share a choice); `refused`: timed candidates dropped because their
        result differed from that of the library's first choice."""
        held, asked, refused = ctypes.c_long(0), ctypes.c_long(0), ctypes.c_long(0)
        self._library().distie_lib_more_counts(ctypes.byref(held), ctypes.byref(asked), ctypes.byref(refused))
        return {"held": held.value, "asked": asked.value, "refused": refused.value}

    LIBRARY_UNSUPPORTED = -3

    def _library_linear(self, x, weight, bias, out_dtype):
        """x [M, K] . weight [N, K]^T (+ float32 bias) by the library, float32 sums, into a new [M, N] of `out_dtype`.
        x and weight are both bfloat16, or both float32 (then every product is a float32 product). None if the
        library has no kernel for the product as asked."""
        M, K = x.shape
        N = weight.shape[0]
        if x.stride(1) != 1 or x.stride(0) != K:
            x = x.contiguous()
        if weight.stride(1) != 1 or weight.stride(0) != K:
            weight = weight.contiguous()
        out = torch.empty((M, N), dtype=out_dtype, device=self.device)
        lib = self._library()
        code, size, w_size = _CODES[out_dtype], out.element_size(), weight.element_size()
        # The library's large bfloat16 kernels work on tiles of 256 x 256, one a compute unit at a time: a product
        # with a few tiles more than a whole number of rounds pays a full round for them (at 2,048 rows 16,384
        # columns take 82 us and 17,920 take 116). The last columns as a product of their own cost less (20 us
        # for 1,536), written into the same output.
        tail = self._library_tail(M, N) if out_dtype == torch.bfloat16 else 0
        for lo, hi in (((0, N - tail), (N - tail, N)) if tail else ((0, N),)):
            rc = lib.distie_lib_linear(
                x.data_ptr(), weight.data_ptr() + lo * K * w_size, bias.data_ptr() + lo * 4 if bias is not None else None,
                out.data_ptr() + lo * size, _code(x), code, M, hi - lo, K, N, 1 if self._tuning else 0, self._stream())
            if rc == self.LIBRARY_UNSUPPORTED:
                return None
            _check(rc, "lib_linear")
        return out

    LIBRARY_TILE = 256

    def _library_tail(self, M: int, N: int) -> int:
        """How many of the last columns of a large library product to run as a product of their own: those
        beyond the last whole round of tiles over the compute units, if they are few (at most a quarter of a
        round) and there is at least one whole round before them; else 0."""
        tile = self.LIBRARY_TILE
        row_tiles = -(-M // tile)
        if row_tiles > self._compute_units:
            return 0
        round_columns = self._compute_units // row_tiles * tile
        tail = N % round_columns
        if N < round_columns or tail == 0 or tail > round_columns // 4 or tail % 8:
            return 0
        return tail

    def _pass_blocks(self, rows: int, elements: int) -> int:
        """Blocks of 16 rows of x per pass of the wide product over a weight of `elements` (0: one pass)."""
        if elements > self.TWO_PASS_MAX_ELEMENTS:
            if rows <= 64:
                return 0
            blocks = -(-rows // 16)
            passes = -(-blocks // self.WIDE_PASS_MAX_BLOCKS)
            return -(-blocks // passes)
        # (a single pass takes at most 64 rows; beyond 128 rows passes of 48 were 5 % faster than of 32 or 64)
        return 0 if rows <= 32 else (2 if rows <= 128 else 3)

    def _rope_table(self, meta, inv_freq):
        """Cosines and sines of the step's positions, float32 [T, pairs, 2]: computed by the first layer
        that asks, used by all."""
        pairs = inv_freq.shape[0]
        key = ("rope", inv_freq.data_ptr(), pairs)
        table = meta.scratch.get(key)
        if table is None:
            table = torch.empty((meta.num_tokens, pairs, 2), dtype=torch.float32, device=self.device)
            _check(self._ops.distie_rope_table(meta.positions.data_ptr(), inv_freq.data_ptr(), table.data_ptr(),
                                               meta.num_tokens, pairs, self._stream()), "rope_table")
            meta.scratch[key] = table
        return table

    def _linear(self, x, weight, bias, out_dtype, partial_ok=False, lazy=False):
        packed = getattr(weight, "_distie_packed", None)
        if isinstance(x, PendingNorm) and out_dtype == torch.float32 and bias is None and packed is not None and \
                weight.shape[1] == x.shape[1] and weight.dtype == torch.bfloat16:
            # the head behind the final norm
            N, K = weight.shape
            if packed.numel() != self._packed_elements(N, K, False):
                raise KernelError("linear: the packed copy does not belong to this weight")
            out = torch.empty((x.shape[0], N), dtype=torch.float32, device=self.device)
            return self._norm_product(x, packed, None, out, 0, N)
        x = self.dense(x)
        self._own(x, weight, bias)
        M, K = x.shape
        N = weight.shape[0]
        if weight.shape[1] != K:
            raise KernelError(f"linear: x is [{M}, {K}], weight is {list(weight.shape)}")
        if bias is not None and (bias.dtype != torch.float32 or bias.shape[0] != N):
            raise KernelError("linear: bias must be float32 [N]")
        both_bf16 = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
        packed = packed if both_bf16 else None
        if lazy and packed is not None and self._fused(M) and K % 8 == 0 and out_dtype == torch.bfloat16:
            return PendingProduct(x, weight, bias)
        if packed is not None and self.ONE_WAVE_MAX_ROWS < M <= self._packed_rows(M, N, K) and K % 8 == 0 and \
                N * K > self.ROW_GROUPS_MAX_ELEMENTS:
            if packed.numel() != self._packed_elements(N, K, False):
                raise KernelError("linear: the packed copy does not belong to this weight")
            slices = self._ops.distie_gemm_packed_wide_slices(N, K)
            if slices == 1:
                out = torch.empty((M, N), dtype=out_dtype, device=self.device)
            else:
                out = torch.empty((slices, M, N), dtype=torch.float32, device=self.device)
            _check(self._ops.distie_gemm_packed_wide_bf16(
                x.data_ptr(), packed.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
                _code(out), M, N, K, 0, self._pass_blocks(M, N * K), self._stream()),
                "gemm_packed_wide_bf16")
            if slices == 1:
                return out
            return PartialSums(out, out_dtype) if partial_ok else self.dense(PartialSums(out, out_dtype))
        if both_bf16 and K % 8 == 0 and (M <= self.SKINNY_MAX_ROWS or (packed is not None and M <= self._packed_rows(M, N, K))):
            if packed is not None:
                if packed.numel() != self._packed_elements(N, K, False):
                    raise KernelError("linear: the packed copy does not belong to this weight")
            slices = self._ops.distie_gemm_skinny_slices(M, N, K)       # the same cut for both kernels
            if slices == 1:
                out = torch.empty((M, N), dtype=out_dtype, device=self.device)
            else:
                out = torch.empty((slices, M, N), dtype=torch.float32, device=self.device)
            if packed is not None:
                _check(self._ops.distie_gemm_packed_bf16(
                    x.data_ptr(), packed.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
                    _code(out), M, N, K, 0, self._stream()), "gemm_packed_bf16")
            else:
                _check(self._ops.distie_gemm_skinny_bf16(
                    x.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
                    _code(out), M, N, K, self._stream()), "gemm_skinny_bf16")
            if slices == 1:
                return out
            return PartialSums(out, out_dtype) if partial_ok else self.dense(PartialSums(out, out_dtype))
        if both_bf16:
            # large bfloat16 product: the library's matrix-core kernels
            out = self._library_linear(x, weight, bias, out_dtype)
            if out is None:
                # no kernel of the library's for this product as asked for: through torch, which knows more ways
                out = torch.mm(x, weight.t(), out_dtype=torch.float32)
                out = out if bias is None else out + bias
                out = out if out_dtype == torch.float32 else out.to(out_dtype)
            return out
        both_f32 = x.dtype == torch.float32 and weight.dtype == torch.float32 and out_dtype == torch.float32
        if both_f32 and M > self.ROWS_MAX_ROWS:
            # large float32 product: the library's float32 kernels (float32 products and sums); else the generic one
            out = self._library_linear(x, weight, bias, out_dtype)
            if out is not None:
                return out
        out = torch.empty((M, N), dtype=out_dtype, device=self.device)
        if M <= self.ROWS_MAX_ROWS and K % 8 == 0:
            # few rows in float32 (or against a weight kept in float32): the weights are streamed, FMAs only
            _check(self._ops.distie_gemv_rows(
                x.data_ptr(), _code(x), weight.data_ptr(), _code(weight), bias.data_ptr() if bias is not None else None,
                out.data_ptr(), _CODES[out_dtype], M, N, K, self._stream()), "gemv_rows")
            return out
        _check(self._ops.distie_gemm_generic(
            x.data_ptr(), _code(x), weight.data_ptr(), _code(weight), bias.data_ptr() if bias is not None else None,
            out.data_ptr(), _CODES[out_dtype], M, N, K, self._stream()), "gemm_generic")
        return out

    def linear(self, x, weight, bias=None):
        """May return `PartialSums` (see there)."""
        return self._linear(x, weight, bias, x.dtype, partial_ok=True, lazy=True)

    def linear_f32out(self, x, weight):
        return self._linear(x, weight, None, torch.float32)

    def rope_kv_write(self, qkv, meta: BatchMeta, group, k_cache, v_cache, inv_freq, num_heads, num_kv_heads,
                      head_dim, write):
        if isinstance(qkv, (PendingNorm, PendingProduct)):
            qkv = self.dense(qkv)
        slices, source = 1, qkv
        if isinstance(qkv, PartialSums):
            slices, source = qkv.slices, qkv.data
            out = torch.empty(tuple(qkv.shape), dtype=qkv.dtype, device=self.device)
        else:
            out = qkv
        self._own(source, k_cache, v_cache, inv_freq)
        T = out.shape[0]
        if out.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
            raise KernelError("rope_kv_write: qkv width does not match the head counts")
        self._check_cache(k_cache, v_cache, num_kv_heads, meta.block_size, head_dim)
        if T != meta.num_tokens:
            raise KernelError("rope_kv_write: qkv rows do not match the batch")
        pairs = 0 if inv_freq is None else inv_freq.shape[0]
        slots = meta.groups[group].slots
        table = self._rope_table(meta, inv_freq) if pairs else None
        _check(self._ops.distie_rope_kv_write(
            source.data_ptr(), _code(source), slices, out.data_ptr(), _code(out),
            table.data_ptr() if table is not None else None, meta.positions.data_ptr(),
            slots.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), _code(k_cache),
            inv_freq.data_ptr() if inv_freq is not None else None, pairs, T, num_heads, num_kv_heads, head_dim,
            meta.block_size, 1 if write else 0, self._stream()), "rope_kv_write")
        _mark_written(out)
        return out

    def paged_attention(self, qkv, meta: BatchMeta, group, k_cache, v_cache, num_heads, num_kv_heads, head_dim,
                        scale, window, extras=None):
        """The matrix-core kernels and the tiled float32 kernel compute plain attention; a step with
        `extras` goes to the wave-per-token kernel, which takes slopes and a cap (any types and sizes)."""
        if not scale > 0:
            raise KernelError(f"paged_attention: the scale of the scores must be positive, not {scale}")
        qkv = self.dense(qkv)
        self._own(qkv, k_cache, v_cache)
        lib = self.attention_library(head_dim)
        T = qkv.shape[0]
        table = meta.groups[group].block_table
        self._check_cache(k_cache, v_cache, num_kv_heads, meta.block_size, head_dim)
        rows = meta.table_rows
        if T != meta.num_tokens or (rows is None and table.shape[0] != meta.num_requests) or \
                (rows is not None and rows.shape[0] != meta.num_requests):
            raise KernelError("paged_attention: tensors do not match the batch")
        rows_ptr = rows.data_ptr() if rows is not None else None
        out = torch.empty((T, num_heads * head_dim), dtype=qkv.dtype, device=self.device)
        plain = extras is None or extras.plain
        slopes, cap = (None, 0.0) if plain else (extras.head_slopes, float(extras.score_cap or 0.0))
        if slopes is not None:
            self._own(slopes)
            if slopes.dtype != torch.float32 or tuple(slopes.shape) != (num_heads,):
                raise KernelError("paged_attention: head_slopes must be float32 [num_heads]")
        bf16 = qkv.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16
        if plain and bf16 and meta.block_size % 16 == 0 and head_dim % 16 == 0:
            # how the step is launched, and its buffers for partial results, are the same for every layer
            # with these sizes: worked out once per step (the layers run one after the other, so they can
            # share the buffers)
            key = ("attention", int(window or 0), num_heads, num_kv_heads, head_dim, meta.max_kv, meta.all_decode,
                   meta.singles_bound, self.PREFILL_PARTS, self.PREFILL_WORKGROUPS, self.DECODE_WAVES, self.DECODE_MAX_RUNS,
                   self.DECODE_SHARED_BELOW)
            plan = meta.scratch.get(key)
            if plan is None or plan["cu_q"] is not meta.host_cu_q:
                plan = meta.scratch[key] = self._attention_plan(lib, meta, T, num_heads, num_kv_heads, head_dim, window)
            if plan["decode"]:
                _check(lib.distie_attention_decode_bf16(
                    qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), meta.kv_len.data_ptr(),
                    meta.cu_q.data_ptr(), table.data_ptr(), table.shape[1], rows_ptr, out.data_ptr(),
                    plan["decode_o"].data_ptr(), plan["decode_ml"].data_ptr(), meta.num_requests, num_heads,
                    num_kv_heads, meta.block_size, float(scale), int(window or 0), plan["split_len"],
                    plan["max_splits"], 1 if meta.all_decode else 0,
                    plan["run_len"].data_ptr() if plan["run_len"] is not None else None, self._stream()),
                    "attention_decode_bf16")
            if plan["prefill"]:
                parts = plan["parts"]
                _check(lib.distie_attention_prefill_bf16(
                    qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), meta.positions.data_ptr(),
                    meta.cu_q.data_ptr(), table.data_ptr(), table.shape[1], rows_ptr, out.data_ptr(), T, meta.num_requests,
                    num_heads, num_kv_heads, meta.block_size, float(scale), int(window or 0),
                    2 if plan["decode"] else 1, meta.token_request.data_ptr(),
                    plan["prefill_o"].data_ptr() if parts > 1 else None,
                    plan["prefill_ml"].data_ptr() if parts > 1 else None, parts, self._stream()),
                    "attention_prefill_bf16")
            return out
        f32 = qkv.dtype == torch.float32 and k_cache.dtype == torch.float32
        if plain and f32 and meta.max_q >= self.PREFILL_F32_MIN_TOKENS and meta.block_size % 16 == 0 and \
                qkv.shape[1] % 4 == 0 and lib.distie_attention_prefill_f32_fits():
            # portions of prompts in float32: the tiled kernel on float32 matrix products takes the whole step
            key = ("attention_f32", int(window or 0), num_heads, head_dim, meta.max_kv, self.PREFILL_PARTS,
                   self.PREFILL_WORKGROUPS)
            plan = meta.scratch.get(key)
            if plan is None:
                plan = meta.scratch[key] = self._prefill_parts(meta, T, num_heads, head_dim, window)
            parts = plan["parts"]
            _check(lib.distie_attention_prefill_f32(
                qkv.data_ptr(), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), meta.positions.data_ptr(),
                meta.cu_q.data_ptr(), table.data_ptr(), table.shape[1], rows_ptr, out.data_ptr(), T, meta.num_requests,
                num_heads, num_kv_heads, meta.block_size, float(scale), int(window or 0), 1,
                meta.token_request.data_ptr(), plan["prefill_o"].data_ptr() if parts > 1 else None,
                plan["prefill_ml"].data_ptr() if parts > 1 else None, parts, self._stream()), "attention_prefill_f32")
            return out
        _check(lib.distie_attention_generic(
            qkv.data_ptr(), _code(qkv), qkv.shape[1], k_cache.data_ptr(), v_cache.data_ptr(), _code(k_cache),
            meta.positions.data_ptr(), meta.token_request.data_ptr(), table.data_ptr(), table.shape[1], rows_ptr,
            out.data_ptr(), T, num_heads, num_kv_heads, meta.block_size, float(scale), int(window or 0),
            slopes.data_ptr() if slopes is not None else None, cap, self._stream()), "attention_generic")
        return out

    def _attention_plan(self, lib, meta: BatchMeta, T, num_heads, num_kv_heads, head_dim, window) -> dict:
        group = num_heads // num_kv_heads
        singles = meta.num_requests if meta.all_decode else 0
        if not meta.all_decode and meta.singles_bound is not None:
            # a captured step of portions and single tokens: which requests bring one token is known on the device
            # only; both kernels are launched for as many as there may be, and each leaves the other's requests alone
            singles = meta.singles_bound
        elif not meta.all_decode and meta.host_cu_q is not None:
            singles = int((meta.host_cu_q[1:] - meta.host_cu_q[:-1] == 1).sum())
        plan = {"cu_q": meta.host_cu_q, "decode": singles > 0 and group <= lib.distie_attention_decode_columns()}
        if plan["decode"]:
            # requests that bring one token: keys are cut into runs, one wave each, so that the chip is
            # filled even when few requests decode. The kernel cuts every request's visible keys (counted
            # from a 64-key boundary) into at most `max_splits` runs by the request's own length; the length
            # of the longest request's runs is passed along as a hint for the first lookups of pages.
            visible = min(meta.max_kv, int(window) + 63) if window else meta.max_kv
            max_splits = max(1, min(self.DECODE_MAX_RUNS, self.DECODE_WAVES // (singles * num_kv_heads),
                                    -(-visible // 64)))
            plan["split_len"] = -(-visible // (64 * max_splits)) * 64
            # every request with one token, no window, waves left over: one run length for all of them, so that a
            # long request gets more runs than a short one (up to twice what every request would get)
            plan["run_len"] = None
            pairs = singles * num_kv_heads
            if meta.all_decode and not window and max_splits * pairs <= self.DECODE_SHARED_BELOW * self.DECODE_WAVES:
                splits = max_splits
                max_splits = max(1, min(self.DECODE_MAX_RUNS, 2 * splits, -(-visible // 64)))
                plan["run_len"] = torch.empty(1, dtype=torch.int32, device=self.device)
                _check(lib.distie_attention_decode_run_len(meta.kv_len.data_ptr(), meta.num_requests,
                                                           max(1, self.DECODE_WAVES // num_kv_heads), max_splits,
                                                           plan["run_len"].data_ptr(), self._stream()),
                       "attention_decode_run_len")
            plan["max_splits"] = max_splits
            plan["decode_o"] = torch.empty((meta.num_requests, num_heads, max_splits, head_dim), dtype=torch.float32,
                                           device=self.device)
            plan["decode_ml"] = torch.empty((meta.num_requests, num_heads, max_splits, 2), dtype=torch.float32,
                                            device=self.device)
        plan["prefill"] = singles < meta.num_requests or not plan["decode"] or \
            (meta.singles_bound is not None and not meta.all_decode)
        if plan["prefill"]:
            plan.update(self._prefill_parts(meta, T, num_heads, head_dim, window))
        return plan

    def _prefill_parts(self, meta: BatchMeta, T, num_heads, head_dim, window) -> dict:
        """Into how many parts the tiled kernel cuts its walk over the keys, and the buffers between it and the
        merge. Portions of prompts (and single tokens too, if no other kernel took them): long walks over the
        keys are cut into parts that run side by side."""
        visible = min(meta.max_kv, int(window) + 128) if window else meta.max_kv
        parts = 1
        for keys, cut in self.PREFILL_PARTS:
            if visible >= keys:
                parts = cut
        # few new tokens make few workgroups (one per 128 tokens of a request and head), each walking all
        # the keys alone: more parts then, down to 128 keys a part
        tiles = -(-T // 128) + meta.num_requests
        wanted = -(-self.PREFILL_WORKGROUPS // (tiles * num_heads))
        parts = max(parts, min(wanted, visible // 128, 16))
        plan = {"parts": parts}
        if parts > 1:
            plan["prefill_o"] = torch.empty((parts, T, num_heads, head_dim), dtype=torch.float32, device=self.device)
            plan["prefill_ml"] = torch.empty((parts, T, num_heads, 2), dtype=torch.float32, device=self.device)
        return plan

    def silu_mul(self, gate_up):
        if isinstance(gate_up, (PendingNorm, PendingProduct)):
            gate_up = self.dense(gate_up)
        slices, source, dtype = 1, gate_up, gate_up.dtype
        if isinstance(gate_up, PartialSums):
            slices, source = gate_up.slices, gate_up.data
        self._own(source)
        rows, two = gate_up.shape
        out = torch.empty((rows, two // 2), dtype=dtype, device=self.device)
        _check(self._ops.distie_silu_mul(source.data_ptr(), _code(source), slices, out.data_ptr(), _code(out),
                                         rows, two // 2, self._stream()), "silu_mul")
        return out

    def gather_rows(self, x, rows):
        x = self.dense(x)
        self._own(x, rows)
        out = torch.empty((rows.shape[0], x.shape[1]), dtype=x.dtype, device=self.device)
        _check(self._ops.distie_gather_rows(x.data_ptr(), rows.data_ptr(), out.data_ptr(), rows.shape[0],
                                            x.shape[1] * x.element_size(), x.shape[0], self._stream()), "gather_rows")
        return out

    def argmax(self, logits):
        self._own(logits)
        if logits.dtype != torch.float32:
            raise KernelError("argmax reads float32 logits")
        rows, vocab = logits.shape
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        parts = self._ops.distie_argmax_parts(rows, vocab)
        values = indexes = None
        if parts > 1:
            values = torch.empty(rows * parts, dtype=torch.float32, device=self.device)
            indexes = torch.empty(rows * parts, dtype=torch.int32, device=self.device)
        _check(self._ops.distie_argmax(logits.data_ptr(), out.data_ptr(), rows, vocab,
                                       values.data_ptr() if parts > 1 else None,
                                       indexes.data_ptr() if parts > 1 else None, self._stream()), "argmax")
        return out

    def sample(self, logits, temperature, seeds, counters):
        self._own(logits, temperature, seeds, counters)
        if logits.dtype != torch.float32 or temperature.dtype != torch.float32 or \
                seeds.dtype != torch.int64 or counters.dtype != torch.int64:
            raise KernelError("sample: logits/temperature float32, seeds/counters int64")
        rows, vocab = logits.shape
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        parts = self._ops.distie_argmax_parts(rows, vocab)
        values = indexes = sums = None
        if parts > 1:
            values = torch.empty(rows * parts, dtype=torch.float32, device=self.device)
            indexes = torch.empty(rows * parts, dtype=torch.int32, device=self.device)
            sums = torch.empty(rows * parts, dtype=torch.float32, device=self.device)
        _check(self._ops.distie_sample(logits.data_ptr(), temperature.data_ptr(), seeds.data_ptr(),
                                       counters.data_ptr(), out.data_ptr(), rows, vocab,
                                       values.data_ptr() if parts > 1 else None,
                                       indexes.data_ptr() if parts > 1 else None,
                                       sums.data_ptr() if parts > 1 else None, self._stream()), "sample")
        return out
