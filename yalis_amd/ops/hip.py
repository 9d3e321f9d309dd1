"""The kernel library: ctypes bindings of the HIP kernels in ``yalis_amd/csrc``.

Every method takes torch tensors on the GPU, checks what the kernels assume, and
launches on torch's current stream.  There is no other implementation behind these
methods: when the library cannot be built or loaded, constructing ``HipOps``
raises.  Plain matrix products of many rows in bfloat16 go to the vendor library
(hipBLASLt, called from ``csrc/library_gemm.hip``; the reference uses cuBLAS in the same
places, yalis/external/model.py:449,462-466,717-722); few-row products, every float32
product and everything else are the hand-written kernels.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from .build import load_kernels

_F32, _BF16 = 0, 1
_c_int = ctypes.c_int
_c_float = ctypes.c_float
_c_size_t = ctypes.c_size_t
_vp = ctypes.c_void_p


class KernelError(RuntimeError):
    pass


class StaleWorkspace(KernelError):
    """A result that lives in the library's workspace was consumed after the workspace had
    been handed to a later launch."""


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"kernels take float32 and bfloat16 only, got {dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_SIGNATURES = {
    "yk_abi_version": ([], _c_int),
    "yk_cache_tiled": ([_c_int, _c_int, _c_int], _c_int),
    "yk_embed": ([_vp, _vp, _c_int, _vp, _c_int, _c_int, _c_int, _vp], _c_int),
    "yk_add_rmsnorm": (
        [_vp, _vp, _c_int, _c_int, _c_int, _vp, _vp, _c_int, _vp, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _vp, _c_int, _vp],
        _c_int,
    ),
    "yk_rope_append": (
        [_vp, _c_int, _c_int, _c_int, _c_int, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _vp, _vp,
         _c_int, _c_int, _c_int, _vp, _vp, _vp, _c_int, _vp],
        _c_int,
    ),
    "yk_add_bias": ([_vp, _c_int, _c_int, _vp, _c_int, _c_int, _vp, _c_int, _c_int, _c_int, _vp], _c_int),
    "yk_gated_act": ([_vp, _c_int, _c_int, _c_int, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp], _c_int),
    "yk_gemm_fma": (
        [_vp, _c_int, _vp, _c_int, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp],
        _c_int,
    ),
    "yk_gemm_skinny_splits": ([_c_int, _c_int, _c_int, _c_int], _c_int),
    "yk_gemm_skinny_force": ([_c_int, _c_int, _c_int], _c_int),
    "yk_gemm_skinny_wide": ([_c_int], _c_int),
    "yk_gemm_library": ([_vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_size_t, _vp, _vp], _c_int),
    "yk_gemm_library_tune": ([_c_int], _c_int),
    "yk_gemm_mfma_skinny": (
        [_vp, _vp, _vp, _c_int, _vp, _c_size_t, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp],
        _c_int,
    ),
    "yk_gemm_tile": (
        [_vp, _vp, _vp, _c_int, _vp, _c_size_t, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp],
        _c_int,
    ),
    "yk_gemm_tile_splits": ([_c_int, _c_int, _c_int], _c_int),
    "yk_gemm_tile_force": ([_c_int], _c_int),
    "yk_attn_generic": (
        [_vp, _c_int, _vp, _vp, _vp, _c_int, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _vp],
        _c_int,
    ),
    "yk_attn_mfma_supported": ([_c_int], _c_int),
    "yk_attn_heads_per_tile": ([_c_int, _c_int], _c_int),
    "yk_attn_long_tile_tokens": ([_c_int, _c_int, _c_int], _c_int),
    "yk_attn_tokens_per_tile": ([_c_int, _c_int], _c_int),
    "yk_attn_mfma_workspace": ([_c_int, _c_int, _c_int, _c_int, _c_int], _c_size_t),
    "yk_attn_mfma_prefill": (
        [_vp, _c_int, _vp, _vp, _vp, _vp, _c_int, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _vp, _c_size_t, _c_int, _vp],
        _c_int,
    ),
    "yk_attn_mfma": (
        [_vp, _c_int, _vp, _vp, _vp, _vp, _c_int, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _vp, _c_size_t, _c_int, _vp],
        _c_int,
    ),
    "yk_attn_mfma_rope": (
        [_vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _vp, _vp, _vp, _vp, _c_int,
         _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _vp, _c_size_t, _c_int, _vp],
        _c_int,
    ),
    "yk_attn_combine": ([_vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_size_t, _vp], _c_int),
    "yk_gemm_skinny_from_attention_ok": ([_c_int, _c_int, _c_int], _c_int),
    "yk_gemm_mfma_skinny_from_attention": (
        [_vp, _c_size_t, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _vp, _c_int, _vp, _c_size_t, _c_int, _c_int, _c_int, _c_int, _c_int, _vp],
        _c_int,
    ),
}
# the libraries that are built and loaded when first used (choosing tokens; the benchmark's probes)
_LATER_SIGNATURES = {
    "sampling": {
        "yk_abi_version": ([], _c_int),
        "yk_argmax": ([_vp, _vp, _c_int, _c_int, _vp, _c_size_t, _vp], _c_int),
        "yk_sample": ([_vp, _vp, _c_int, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int, _vp, _c_size_t, _vp, _vp], _c_int),
        "yk_sample_workspace_bytes": ([_c_int, _c_int], _c_size_t),
    },
    "probe": {
        "yk_abi_version": ([], _c_int),
        "yk_probe_stream_read": ([_vp, _c_size_t, _c_int, _c_int, _vp, _vp], _c_int),
        "yk_probe_mfma_bf16": ([_c_int, _c_int, _vp, _vp], _c_int),
    },
}
_ABI = 16

# Rows of x up to which the hand-written matrix-core kernel runs a bfloat16 product;
# above it the vendor library does.
SKINNY_MAX_ROWS = 64
# Waves the attention launch aims at when it decides how far to split the keys.
ATTN_TARGET_WAVES = 1024
# Tokens of a step up to which an attention leaves its splits unmerged for the product that
# follows.  Every workgroup of that product merges its own slice of them again, so the saved
# kernel pays for few tokens only.  Measured at the 8B shape, 1,024-token contexts (ms a step,
# merged by a kernel of its own / by the product): 1 token 3.439 / 3.381, 2 tokens 3.471 /
# 3.427, 3 tokens 3.505 / 3.499, 4 tokens 3.506 / 3.526, 8 tokens 3.635 / 3.695.  The kernel
# takes up to 16.
MERGE_IN_PRODUCT_MAX_TOKENS = 2


class SplitSum:
    """The unreduced K slices of a product: float32 [slices, rows, columns] whose sum over
    the first axis is the result.  The kernels that consume a projection (norm, rotary +
    append, gated activation) add the slices themselves, which saves a pass over memory
    of its own.  ``out_dtype`` is the dtype the product was asked for: the consumers round
    the sum to it, so that a value does not depend on whether its product came reduced or
    as slices.  It lives in the library's workspace: consume it before the next product
    is launched.  One that the library made carries the workspace's generation number, and
    the library refuses (``StaleWorkspace``) to consume it once a later product has taken
    the workspace."""

    def __init__(self, tensor: torch.Tensor, out_dtype: torch.dtype = torch.float32, owner=None, generation: int = 0):
        self.tensor = tensor
        self.owner, self.generation = owner, generation
        self.shape = tuple(tensor.shape[1:])
        self.n_splits = tensor.shape[0]
        self.out_dtype = out_dtype
        self.dtype = torch.float32
        self.device = tensor.device

    @property
    def round_sum(self) -> int:
        return int(self.out_dtype == torch.bfloat16)

    def check_live(self) -> None:
        if self.owner is not None and self.generation != self.owner._gemm_gen:
            raise StaleWorkspace(
                "a product's unreduced slices (SplitSum) were consumed after a later product had been launched: the "
                "library's workspace holds that product's slices now.  Consume a linear(..., partial_ok=True) result "
                "(norm, rotary + append, gated activation, .reduce()) before the next linear, or ask without partial_ok")

    def reduce(self) -> torch.Tensor:
        """The product itself, float32 (for code that does not add the slices itself)."""
        self.check_live()
        return self.tensor.sum(0).to(self.out_dtype).float()

    def float(self) -> torch.Tensor:
        return self.reduce()


class EmbeddedRows:
    """The rows of an embedding table that a step's tokens name, not yet gathered: it stands
    for a tensor [tokens, width] with which a residual stream starts.  The norm kernel that
    comes first gathers the rows itself (``add_rmsnorm`` with this as ``delta`` fills the
    residual and normalises it in one pass); ``gather()`` gives the tensor (float32)."""

    def __init__(self, ops, token_ids: torch.Tensor, table: torch.Tensor):
        self.ops, self.token_ids, self.table = ops, token_ids, table
        self.shape = (token_ids.numel(), table.shape[1])
        self.dtype = torch.float32
        self.device = table.device

    def gather(self) -> torch.Tensor:
        return self.ops.embed(self.token_ids, self.table)

    def float(self) -> torch.Tensor:
        return self.gather()


class SplitAttention:
    """The output of an attention whose keys were split across workgroups, not yet merged:
    it stands for a bfloat16 tensor [tokens, heads * head_dim].  ``HipOps.linear`` merges the
    splits while it stages them as its input where its kernel can (up to 16 tokens), which
    saves the merging kernel; ``merge()`` gives the tensor itself.  It lives in the library's
    workspace: consume it before the next attention (or anything else that takes that
    workspace: choosing tokens) is launched; the library refuses a stale one."""

    def __init__(self, ops, workspace, tiles, token_cols, n_tokens, n_heads, n_kv, head_dim, n_splits):
        self.ops, self.workspace, self.tiles, self.token_cols = ops, workspace, tiles, token_cols
        self.generation = ops._ws_gen
        self.n_heads, self.n_kv, self.head_dim, self.n_splits = n_heads, n_kv, head_dim, n_splits
        self.shape = (n_tokens, n_heads * head_dim)
        self.dtype = torch.bfloat16
        self.device = workspace.device

    def check_live(self) -> None:
        if self.generation != self.ops._ws_gen:
            raise StaleWorkspace(
                "an attention's unmerged splits (SplitAttention) were consumed after a later launch had taken the "
                "library's workspace; hand them to linear() or merge() before the next attention")

    def merge(self) -> torch.Tensor:
        ops = self.ops
        self.check_live()
        out = torch.empty(self.shape, dtype=self.dtype, device=self.device)
        ops._check(
            ops.lib.yk_attn_combine(
                out.data_ptr(), self.tiles.data_ptr(), self.tiles.shape[0], self.head_dim, self.n_heads, self.n_kv,
                self.n_splits, self.workspace.data_ptr(), self.workspace.numel(), ops._stream(),
            )
        )
        return out


class RopeInLaunch:
    """What ``HipOps.attention`` needs to rotate and append inside its own launch: the float32
    tables [positions, rotary_dim / 2] (None with rotary_dim 0), how pairs are formed, and
    whether the projection's rows hold keys and values to append (False: queries only, the
    pages already hold this step's keys and values)."""

    def __init__(self, cos, sin, rotary_dim: int, interleaved: bool, append: bool):
        self.cos, self.sin, self.rotary_dim, self.interleaved, self.append = cos, sin, int(rotary_dim), bool(interleaved), bool(append)


class HipOps:
    def __init__(self, device: str = "cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError("HipOps needs a GPU: torch.cuda.is_available() is False")
        self.device = torch.device(device)
        self.lib = self._bind(load_kernels(), _SIGNATURES)
        self._later: dict = {}
        self._answers: dict = {}
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        # the quick way to the current stream's handle, where this torch has it
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self._workspace: Optional[torch.Tensor] = None  # attention splits, argmax parts
        self._library_workspace: Optional[torch.Tensor] = None  # the vendor library's scratch
        self._gemm_workspace: Optional[torch.Tensor] = None  # K slices of products
        # how often each workspace has been handed out: what lives in one (SplitSum,
        # SplitAttention) remembers the number and is refused once it has moved on
        self._ws_gen = 0
        self._gemm_gen = 0
        # page ids a workgroup of the long-span attention keeps in LDS (more: looked up in the
        # block table one by one); tests lower it to walk that path with short tables
        self.long_span_pages_in_lds = 2048

    # ------------------------------------------------------------------ helpers
    @staticmethod
    def _bind(lib, signatures):
        lib.yk_last_error.restype = ctypes.c_char_p
        for name, (args, res) in signatures.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = res
        if lib.yk_abi_version() != _ABI:
            raise KernelError("kernel library and bindings disagree; rebuild (python -c 'import __graft_entry__ as g; g.build()')")
        return lib

    def _library(self, name: str):
        """A library beside the step's kernels, built and loaded at its first use."""
        if name not in self._later:
            self._later[name] = self._bind(load_kernels(name), _LATER_SIGNATURES[name])
        return self._later[name]

    def _stream(self) -> int:
        """The raw handle of torch's current stream on this device (asked for at every
        launch: a graph capture switches streams)."""
        if self._raw_stream is not None:
            return self._raw_stream(self._device_index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def _check(self, rc: int, lib=None) -> None:
        if rc != 0:
            raise KernelError((lib or self.lib).yk_last_error().decode())

    def _grown(self, have: Optional[torch.Tensor], floats: int) -> torch.Tensor:
        if have is not None and have.numel() >= floats:
            return have
        if have is not None and torch.cuda.is_current_stream_capturing():
            # kernels already recorded hold the old buffer's address
            raise KernelError(f"a scratch buffer would have to grow to {floats} floats while a graph is being captured; "
                              "reserve_workspaces() before the capture must ask for more")
        return torch.empty(max(floats, 1 << 22), dtype=torch.float32, device=self.device)

    def _ws(self, floats: int) -> torch.Tensor:
        """Float32 scratch that grows and is reused (stream order keeps uses apart)."""
        self._workspace = self._grown(self._workspace, floats)
        self._ws_gen += 1
        return self._workspace

    def _gemm_ws(self, floats: int) -> torch.Tensor:
        self._gemm_workspace = self._grown(self._gemm_workspace, floats)
        self._gemm_gen += 1
        return self._gemm_workspace

    def reserve_workspaces(self, rows: int, products=()) -> None:
        """Make the scratch buffers large enough for steps of ``rows`` tokens before a graph is
        captured (a buffer must not be replaced while a capture is running: that raises).
        ``products``: the (n, k) of the weight matrices the step multiplies ``rows`` rows by; the
        unreduced K slices of each take slices x rows x n floats."""
        need = 1 << 24
        if rows <= SKINNY_MAX_ROWS:
            for n, k in products:
                if k >= 8 and k % 8 == 0:
                    need = max(need, self._ask("yk_gemm_skinny_splits", rows, n, k, 0) * rows * n)
        self._ws(1 << 24)
        self._gemm_ws(need)

    def force_skinny_plan(self, chunk: int = 0, waves: int = 0, slices: int = 0) -> None:
        """For tests and measurements: force the few-row product's chunk length (128 / 256), waves a
        workgroup and number of K slices (0: the library decides); call without arguments to clear."""
        self._check(self.lib.yk_gemm_skinny_force(int(chunk), int(waves), int(slices)))
        self._answers = {k: v for k, v in self._answers.items() if k[0] not in ("yk_gemm_skinny_splits", "yk_gemm_skinny_from_attention_ok")}

    def wide_skinny_products(self, mode: int = 1) -> None:
        """For tests and measurements: when few-row products of 33 to 64 rows run in the wide form
        (32 x 32 x 16 matrix-core products): 0 never, 1 where the library's rule says so (the
        default: an unsliced K of 8,192 and more), 2 always."""
        self._check(self.lib.yk_gemm_skinny_wide(int(mode)))

    def tune_library_products(self, on: bool = True) -> None:
        """Whether new shapes of up to 256 rows get the vendor library's first candidate (the
        default: the same choice, and the same bits, in every process) or the fastest of its
        candidates, timed when the shape is first met (the choice then depends on the run)."""
        self._check(self.lib.yk_gemm_library_tune(int(bool(on))))

    def workspaces(self):
        """The scratch buffers in use, for whoever must keep them alive (a captured graph)."""
        return (self._workspace, self._gemm_workspace)

    def _ask(self, name: str, *args: int) -> int:
        """A size question to the library (tile sizes, slices, workspace needs): the answers
        depend on the arguments alone, so each is asked once."""
        key = (name, args)
        got = self._answers.get(key)
        if got is None:
            got = self._answers[key] = getattr(self.lib, name)(*args)
        return got

    @staticmethod
    def _rows(t: torch.Tensor, what: str) -> None:
        if t.dim() != 2 or t.stride(1) != 1:
            raise KernelError(f"{what}: expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")

    # ---------------------------------------------------------- sizes a part may ask
    def check_attention_sizes(self, n_heads: int, n_kv: int, head_dim: int, page_size: int) -> None:
        if n_heads % n_kv:
            raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv} kv heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise KernelError(f"attention: head_dim must be a multiple of 16 between 16 and 256, got {head_dim}")
        if page_size % 16:
            raise KernelError(f"attention: page_size must be a multiple of 16, got {page_size}")

    def attention_tokens_per_tile(self, n_heads: int, n_kv: int) -> int:
        return self._ask("yk_attn_tokens_per_tile", n_heads, n_kv)

    def attention_long_span_tile(self, n_heads: int, n_kv: int, col_tiles: int = 1) -> int:
        """Tokens per tile of the kernel for long spans (one workgroup a tile) when a wave
        has ``col_tiles`` (1 or 2) column tiles."""
        return self._ask("yk_attn_long_tile_tokens", n_heads, n_kv, col_tiles)

    @staticmethod
    def attention_long_col_tiles(workgroups: int, fewest_keys: int) -> int:
        """Column tiles per wave for a step's long spans.  ``workgroups``: how many the
        larger tiles (two column tiles a wave) would make; ``fewest_keys``: the fewest keys
        any of the spans has cached before it.  Two where those workgroups fill the GPU twice
        over, or where no span starts from nothing: every block of keys staged through LDS
        then serves twice the columns, and where the tiles are few the keys are split across
        workgroups (``attention_long_splits``).  One for prompts from nothing: they have tiles
        with a few keys and tiles with all of them, which small tiles balance better.
        Measured on the 8B shape (us, one / two, each with its own splits): a whole 2,048-token
        prompt 70 / 77, a whole 4,096-token one 232 / 204, 2,048 tokens against 6,144 cached
        396 / 318, four 512-token portions against 3,584 cached 228 / 182, a 480-token portion
        against 3,616 cached 72 / 65, against 7,200 cached 116 / 103, two such portions
        124 / 111."""
        return 2 if workgroups >= 1024 or fewest_keys >= 1024 else 1

    # ------------------------------------------------------------------ embedding
    def embed(self, token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        self._rows(table, "embed table")
        n = token_ids.numel()
        out = torch.empty((n, table.shape[1]), dtype=torch.float32, device=table.device)
        self._check(
            self.lib.yk_embed(
                token_ids.data_ptr(), table.data_ptr(), _code(table.dtype), out.data_ptr(), n,
                table.shape[1], table.shape[0], self._stream(),
            )
        )
        return out

    def embedded_rows(self, token_ids: torch.Tensor, table: torch.Tensor):
        """(an uninitialised float32 residual [tokens, width], the ``EmbeddedRows`` that the
        first ``add_rmsnorm`` fills it from): the embedding without a kernel of its own."""
        self._rows(table, "embed table")
        residual = torch.empty((token_ids.numel(), table.shape[1]), dtype=torch.float32, device=table.device)
        return residual, EmbeddedRows(self, token_ids, table)

    # ----------------------------------------------------------------------- norm
    def rmsnorm(self, x, weight, eps, unit_offset, out_dtype):
        """norm(x) * weight for rows ``x`` [N, width] that are no residual stream (a tensor, or a
        ``SplitSum`` whose slices are summed on the way); nothing is written but the result."""
        n_splits, round_sum, src = 1, 0, x
        if isinstance(x, SplitAttention):
            x = src = x.merge()
        if isinstance(x, SplitSum):
            x.check_live()
            n_splits, round_sum, src = x.n_splits, x.round_sum, x.tensor
        else:
            self._rows(x, "norm input")
            if not x.is_contiguous():
                raise KernelError("norm input must be contiguous")
        n, width = x.shape
        if weight.numel() != width:
            raise KernelError(f"norm weight has {weight.numel()} elements, rows have {width}")
        out = torch.empty((n, width), dtype=out_dtype, device=src.device)
        self._check(
            self.lib.yk_add_rmsnorm(
                None, src.data_ptr(), _code(src.dtype), n_splits, round_sum, None, weight.data_ptr(), _code(weight.dtype),
                out.data_ptr(), _code(out_dtype), n, n, width, float(eps), int(bool(unit_offset)), None, 0, self._stream(),
            )
        )
        return out

    def _norm(self, residual, delta, rows, weight, eps, unit_offset, out_dtype, n_out):
        self._rows(residual, "residual")
        if residual.dtype != torch.float32 or not residual.is_contiguous():
            raise KernelError("the residual stream must be contiguous float32")
        width = residual.shape[1]
        if weight.numel() != width:
            raise KernelError(f"norm weight has {weight.numel()} elements, rows have {width}")
        n_splits, round_sum = 1, 0
        table_ids, table_rows = None, 0
        if isinstance(delta, EmbeddedRows):
            if rows is not None or tuple(delta.shape) != tuple(residual.shape):
                raise KernelError(f"embedded rows {tuple(delta.shape)} start a residual of their own shape, got {tuple(residual.shape)}")
            table_ids, delta = delta.token_ids, delta.table
            self._rows(delta, "embedding table")
            if not delta.is_contiguous() or table_ids.dtype != torch.int32:
                raise KernelError("the embedding table must be contiguous and the token ids int32")
            table_rows = delta.shape[0]
        elif isinstance(delta, SplitSum):
            delta.check_live()
            n_splits, round_sum, delta = delta.n_splits, delta.round_sum, delta.tensor
            if tuple(delta.shape[1:]) != tuple(residual.shape):
                raise KernelError(f"delta {tuple(delta.shape[1:])} does not match the residual {tuple(residual.shape)}")
        elif delta is not None and (tuple(delta.shape) != tuple(residual.shape) or not delta.is_contiguous()):
            raise KernelError(f"delta {tuple(delta.shape)} does not match the residual {tuple(residual.shape)}")
        out = torch.empty((n_out, width), dtype=out_dtype, device=residual.device)
        self._check(
            self.lib.yk_add_rmsnorm(
                residual.data_ptr(), _ptr(delta), 0 if delta is None else _code(delta.dtype), n_splits, round_sum,
                _ptr(rows), weight.data_ptr(), _code(weight.dtype), out.data_ptr(), _code(out_dtype),
                n_out, residual.shape[0], width, float(eps), int(bool(unit_offset)), _ptr(table_ids), table_rows,
                self._stream(),
            )
        )
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, unit_offset, out_dtype):
        return self._norm(residual, delta, None, weight, eps, unit_offset, out_dtype, residual.shape[0])

    def gather_add_rmsnorm(self, residual, delta, rows, weight, eps, unit_offset, out_dtype):
        return self._norm(residual, delta, rows, weight, eps, unit_offset, out_dtype, rows.numel())

    # --------------------------------------------------------------------- linear
    def linear(self, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, partial_ok: bool = False, bias=None):
        """x [M, K] . w [N, K]^T (+ bias [N]) -> [M, N].  With ``partial_ok`` (and no bias) the
        result may come as a ``SplitSum`` for a consumer that adds the slices itself."""
        if bias is not None:
            # the product in float32, the bias added there, one rounding (as a product that adds
            # the bias to its accumulators rounds: the reference's biased Linear)
            acc = self.linear(x, w, torch.float32, partial_ok=False)
            if bias.numel() != acc.shape[1] or not bias.is_contiguous():
                raise KernelError(f"linear: bias has {bias.numel()} elements, the product {acc.shape[1]} columns")
            y = acc if out_dtype == torch.float32 else torch.empty(acc.shape, dtype=out_dtype, device=acc.device)
            if y.shape[0]:
                self._check(self.lib.yk_add_bias(acc.data_ptr(), _code(acc.dtype), acc.stride(0), y.data_ptr(), _code(y.dtype),
                                                 y.stride(0), bias.data_ptr(), _code(bias.dtype), y.shape[0], y.shape[1],
                                                 self._stream()))
            return y
        if isinstance(x, SplitAttention):
            y = self._linear_from_attention(x, w, out_dtype, partial_ok)
            if y is not None:
                return y
            x = x.merge()
        self._rows(x, "linear input")
        self._rows(w, "linear weight")
        m, k = x.shape
        n = w.shape[0]
        if w.shape[1] != k:
            raise KernelError(f"linear: input has {k} columns, weight has {w.shape[1]}")
        if m == 0:
            return torch.empty((0, n), dtype=out_dtype, device=x.device)
        bf = torch.bfloat16
        aligned = k % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
        if x.dtype == bf and w.dtype == bf and aligned:
            if out_dtype == bf and self.long_matrix_tiles(m, n, k):
                return self.gemm_tile(x, w, bf, partial_ok)
            if m > SKINNY_MAX_ROWS and out_dtype == bf and not self.few_library_tiles(m, n):
                return self.gemm_library(x, w, bf)  # vendor library, bfloat16 in and out
            if m > SKINNY_MAX_ROWS and out_dtype == torch.float32:
                # vendor library, float32 accumulators stored as they are (the output head for
                # more than 64 wanted rows: the few-row kernel would stream the table once per 64)
                return self.gemm_library(x, w, torch.float32)
            return self.gemm_mfma_skinny(x, w, out_dtype, partial_ok)
        return self.gemm_fma(x, w, out_dtype)

    @staticmethod
    def long_matrix_tiles(m: int, n: int, k: int) -> bool:
        """Whether a product of 65 to 256 rows is ``gemm_tile``'s: where the matrix is at least twice
        as long as it is wide (a down projection), so that tiles of 128 x 128 cut along K occupy
        the GPU and the slices are long.  Measured in replayed graphs (us, vendor library's first
        candidate / few-row kernel / tiles): 8B down-proj (4,096 x 14,336) at 72 rows 36.6 / 37.2 /
        25.6, at 128 57.9 / 35.4 / 27.0, at 192 77.5 / 65.9 / 49.3, at 256 45.9 / - / 47.5; 3B
        (3,072 x 8,192) at 128 32.9 / 19.6 / 17.7, at 192 45.3 / 27.5 / 28.5; 70B (8,192 x 28,672) at
        128 200 / 167 / 110, at 256 314 / - / 200; 1B (2,048 x 8,192) at 192 22.9 / 19.7 / 18.2.  On
        squarer matrices the three are within a tenth of each other up to 128 rows, and from 384
        rows on the library wins everywhere."""
        return SKINNY_MAX_ROWS < m <= 256 and k >= 2 * n and k >= 4096

    @staticmethod
    def few_library_tiles(m: int, n: int) -> bool:
        """Whether a product of 65 to 128 rows is still the few-row kernel's: where the vendor
        library's output tiles (256 columns wide) would be too few to occupy the GPU's 256
        compute units, while the few-row kernel divides K among workgroups.  Measured in replayed
        graphs with the library's fastest candidate (us, few-row kernel / library), 8B shapes at
        128 rows: o-proj 13.8 / 15.3, down-proj 38.7 / 52.1, but qkv 23.7 / 16.6 and gate/up
        96 / 58; at 160 rows o-proj 20.2 / 16.4, down-proj 65.6 / 58.7.  3B shapes at 128 rows:
        o-proj 10.9 / 11.4, down-proj 20.6 / 22.9, qkv 13.7 / 13.2.  So: up to 128 rows and up to
        4,096 columns."""
        return m <= 128 and -(-n // 256) <= 16

    def _linear_from_attention(self, x: "SplitAttention", w: torch.Tensor, out_dtype, partial_ok: bool):
        """The few-row product fed by attention's unmerged splits, or None where it does not
        apply (the caller then merges them first)."""
        x.check_live()
        m, k = x.shape
        n = w.shape[0]
        if (w.dim() != 2 or w.dtype != torch.bfloat16 or w.shape[1] != k or w.stride(1) != 1 or w.stride(0) % 8
                or w.data_ptr() % 16 or not self._ask("yk_gemm_skinny_from_attention_ok", m, n, k)):
            return None
        splits = self._ask("yk_gemm_skinny_splits", m, n, k, 0)
        keep = bool(partial_ok and splits > 1)
        ws = self._gemm_ws(splits * m * n) if splits > 1 else None
        y = None if keep else torch.empty((m, n), dtype=out_dtype, device=w.device)
        rc = self.lib.yk_gemm_mfma_skinny_from_attention(
            x.workspace.data_ptr(), x.workspace.numel(), x.token_cols.data_ptr(), x.tiles.shape[0], x.n_splits,
            x.n_heads, x.n_kv, x.head_dim, w.data_ptr(), _ptr(y), _code(out_dtype), _ptr(ws),
            0 if ws is None else ws.numel(), m, n, w.stride(0), n, int(keep), self._stream(),
        )
        if rc < 0:
            raise KernelError(self.lib.yk_last_error().decode())
        if keep:
            return SplitSum(ws[: rc * m * n].view(rc, m, n), out_dtype, self, self._gemm_gen)  # rc: the slices the launch wrote
        return y

    LIBRARY_WORKSPACE_BYTES = 64 << 20

    def gemm_library(self, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """x [M, K] . w [N, K]^T in the vendor library: bfloat16 operands with 16-byte aligned rows,
        float32 accumulation, the result bfloat16 or float32.  Every shape's algorithm is chosen
        when the shape is first met (the library's first candidate, or with
        ``tune_library_products`` the fastest for up to 256 rows) and kept."""
        m, k = x.shape
        n = w.shape[0]
        if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k or x.stride(1) != 1 or w.stride(1) != 1:
            raise KernelError(f"gemm_library: operands {tuple(x.shape)} {x.dtype} and {tuple(w.shape)} {w.dtype}")
        if self._library_workspace is None:
            self._library_workspace = torch.empty(self.LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=self.device)
        y = torch.empty((m, n), dtype=out_dtype, device=x.device)
        self._check(self.lib.yk_gemm_library(
            x.data_ptr(), w.data_ptr(), y.data_ptr(), _code(out_dtype), m, n, k, x.stride(0), w.stride(0), n,
            self._library_workspace.data_ptr(), self._library_workspace.numel(), None, self._stream()))
        return y

    def gemm_tile(self, x, w, out_dtype, partial_ok: bool = False):
        """x [M, K] . w [N, K]^T in tiles of 128 x 128 on the matrix cores (bfloat16 operands with
        16-byte aligned rows): the kernel for some dozens to a few hundred rows against long
        matrices.  Where its plan cuts K the result comes as a ``SplitSum`` (with ``partial_ok``)
        or is summed here."""
        m, k = x.shape
        n = w.shape[0]
        splits = self._ask("yk_gemm_tile_splits", m, n, k)
        ws = self._gemm_ws(splits * m * n) if splits > 1 else None
        y = None if splits > 1 else torch.empty((m, n), dtype=out_dtype, device=x.device)
        rc = self.lib.yk_gemm_tile(
            x.data_ptr(), w.data_ptr(), _ptr(y), _code(out_dtype), _ptr(ws), 0 if ws is None else ws.numel(),
            m, n, k, x.stride(0), w.stride(0), n, self._stream(),
        )
        if rc < 0:
            raise KernelError(self.lib.yk_last_error().decode())
        if rc == 0:
            return y
        part = SplitSum(ws[: rc * m * n].view(rc, m, n), out_dtype, self, self._gemm_gen)
        return part if partial_ok else part.reduce().to(out_dtype)

    def force_tile_slices(self, slices: int = 0) -> None:
        """For tests and measurements: force the K slices of ``gemm_tile`` (0: the library decides)."""
        self._check(self.lib.yk_gemm_tile_force(int(slices)))
        self._answers = {k: v for k, v in self._answers.items() if k[0] != "yk_gemm_tile_splits"}

    def gemm_fma(self, x, w, out_dtype):
        m, k = x.shape
        n = w.shape[0]
        y = torch.empty((m, n), dtype=out_dtype, device=x.device)
        self._check(
            self.lib.yk_gemm_fma(
                x.data_ptr(), _code(x.dtype), w.data_ptr(), _code(w.dtype), y.data_ptr(), _code(out_dtype),
                m, n, k, x.stride(0), w.stride(0), n, self._stream(),
            )
        )
        return y

    # ---------------------------------------------------------- gate/up + activation
    GATE_UP_GROUP = 8  # rows of the packed matrix alternate: 8 of gate, their 8 of up

    def pack_gate_up(self, w_gate: torch.Tensor, w_up: torch.Tensor) -> Tuple[torch.Tensor, int]:
        """One matrix for both projections and the group size of its row order: 0 = [gate; up];
        8 = eight gate rows, then their eight up rows, and so on, which lets the few-row
        product apply the activation itself (the reference keeps gate and up in one matrix
        with rows interleaved too, yalis/external/model.py:717-722)."""
        inter = w_gate.shape[0]
        g = self.GATE_UP_GROUP
        if w_gate.dtype == torch.bfloat16 and w_up.dtype == torch.bfloat16 and inter % g == 0:
            k = w_gate.shape[1]
            packed = self._rows_apart(2 * inter, k, w_gate.device)
            packed.view(inter // g, 2, g, k)[:, 0].copy_(w_gate.view(inter // g, g, k))
            packed.view(inter // g, 2, g, k)[:, 1].copy_(w_up.view(inter // g, g, k))
            return packed, g
        return torch.cat([w_gate, w_up], dim=0).contiguous(), 0

    # Rows of a streamed bfloat16 matrix that would lie a multiple of 4 KiB apart are kept 128 bytes
    # further apart.  Workgroups of the few-row product that walk all of K in step (gate/up, the
    # output head: their K is not sliced) ask, at every moment, for addresses a whole number of
    # rows apart, and rows 4 KiB apart crowd onto few memory channels.  Up to 32 rows of x the
    # product answers that by starting its workgroups at different places of K; with more rows
    # they must stay in step (they share the staged rows of x through L2: started apart, gate/up
    # at 64 rows went 50 -> 64 us), and the gap between rows does it instead: 8B shape, us, rows 8 KiB
    # apart / 128 bytes more: gate/up at 64 rows of x 52.0 / 45.6, at 48 48.0 / 42.6, the head at 64
    # 221 / 197, at 48 212 / 184; at 32 rows and fewer no difference (42.2 / 43.3, 37.0 / 37.5).  The
    # sliced products (qkv, o-proj, down-proj) are better off without (qkv at 64 rows 14.0 / 15.7),
    # and so are rows of 16 KiB (the 70B shape's gate/up at 64 / 8 rows 196 / 223, 151 / 178): the
    # gap is for rows of 4 and 8 KiB (the 1B shape's head at 64 rows 120 / 110).
    ROW_GAP = 64  # elements

    @staticmethod
    def _rows_crowd(k: int) -> bool:
        return 2 * k in (4096, 8192)

    def _rows_apart(self, rows: int, k: int, device) -> torch.Tensor:
        """An uninitialised bfloat16 [rows, k], its rows 128 bytes further apart where that pays."""
        if self._rows_crowd(k):
            return torch.empty((rows, k + self.ROW_GAP), dtype=torch.bfloat16, device=device)[:, :k]
        return torch.empty((rows, k), dtype=torch.bfloat16, device=device)

    def streamed_matrix(self, w: torch.Tensor) -> torch.Tensor:
        """``w`` as a part should keep it when all it does with it is multiply few rows by it with
        K unsliced (an output head): ``w`` itself, or a copy with its rows 128 bytes further apart
        (see above)."""
        if w.dim() != 2 or w.dtype != torch.bfloat16 or not w.is_contiguous() or not self._rows_crowd(w.shape[1]):
            return w
        out = self._rows_apart(w.shape[0], w.shape[1], w.device)
        out.copy_(w)
        return out

    def gate_up_act(self, x: torch.Tensor, w_gate_up: torch.Tensor, group: int, activation: str, out_dtype: torch.dtype) -> torch.Tensor:
        """act(x . gate^T) * (x . up^T) -> [M, intermediate], ``w_gate_up`` and ``group`` as
        ``pack_gate_up`` gave them.  Few rows of bfloat16 whose product is not split over K
        run as one kernel; otherwise the product, then the activation kernel."""
        act = {"silu": 1, "gelu_tanh": 2}.get(activation)
        if act is None:
            raise KernelError(f"unknown activation {activation!r}")
        self._rows(x, "gate/up input")
        m, k = x.shape
        n = w_gate_up.shape[0]
        bf = torch.bfloat16
        fused = (
            group == self.GATE_UP_GROUP and 0 < m <= SKINNY_MAX_ROWS and x.dtype == bf and w_gate_up.dtype == bf and out_dtype == bf
            and w_gate_up.shape[1] == k and k % 8 == 0 and x.stride(0) % 8 == 0 and w_gate_up.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0 and n % 16 == 0
            and self._ask("yk_gemm_skinny_splits", m, n, k, 1) == 1
        )
        if not fused:
            return self.gated_act(self.linear(x, w_gate_up, out_dtype, partial_ok=True), activation, out_dtype, group=group)
        y = torch.empty((m, n // 2), dtype=bf, device=x.device)
        rc = self.lib.yk_gemm_mfma_skinny(
            x.data_ptr(), w_gate_up.data_ptr(), y.data_ptr(), _code(bf), None, 0,
            m, n, k, x.stride(0), w_gate_up.stride(0), n // 2, 0, act, self._stream(),
        )
        if rc < 0:
            self._check(rc)
        return y

    def gemm_mfma_skinny(self, x, w, out_dtype, partial_ok: bool = False):
        m, k = x.shape
        n = w.shape[0]
        splits = self._ask("yk_gemm_skinny_splits", m, n, k, 0)
        keep = bool(partial_ok and splits > 1)
        ws = self._gemm_ws(splits * m * n) if splits > 1 else None
        y = None if keep else torch.empty((m, n), dtype=out_dtype, device=x.device)
        rc = self.lib.yk_gemm_mfma_skinny(
            x.data_ptr(), w.data_ptr(), _ptr(y), _code(out_dtype), _ptr(ws), 0 if ws is None else ws.numel(),
            m, n, k, x.stride(0), w.stride(0), n, int(keep), 0, self._stream(),
        )
        if rc < 0:
            raise KernelError(self.lib.yk_last_error().decode())
        if keep:
            return SplitSum(ws[: rc * m * n].view(rc, m, n), out_dtype, self, self._gemm_gen)  # rc: the slices the launch wrote
        return y

    # ------------------------------------------------- rotary + append to the cache
    def rope_append(self, qkv, n_heads, n_kv, head_dim, positions, cos, sin, rotary_dim,
                    interleaved, k_cache, v_cache, slots, page_size) -> torch.Tensor:
        """Rotates the query heads, appends rotated keys and values to the pages; returns
        the tensor whose rows start with the rotated queries (``qkv`` itself, rotated in
        place, or a new [N, n_heads * head_dim] tensor when ``qkv`` is a SplitSum)."""
        n_splits, round_sum = 1, 0
        src = qkv
        if isinstance(qkv, SplitSum):
            qkv.check_live()
            n_splits, round_sum, src = qkv.n_splits, qkv.round_sum, qkv.tensor
            n, cols = qkv.shape
            act = k_cache.dtype if n_kv else torch.bfloat16
            q_out = torch.empty((n, n_heads * head_dim), dtype=act, device=src.device)
            src_stride = cols
        else:
            self._rows(qkv, "qkv")
            n, cols = qkv.shape
            q_out = qkv
            src_stride = qkv.stride(0)
        if cols != (n_heads + 2 * n_kv) * head_dim:
            raise KernelError(f"qkv rows have {cols} elements, expected {(n_heads + 2 * n_kv) * head_dim}")
        if positions.numel() != n or (n_kv > 0 and slots.numel() != n):
            raise KernelError("positions/slots do not match the number of tokens")
        max_pos = 0
        if rotary_dim:
            if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rotary_dim // 2:
                raise KernelError("rotary tables must be float32 [positions, rotary_dim/2]")
            max_pos = cos.shape[0]
        if n_kv > 0:
            if k_cache.dtype != q_out.dtype or v_cache.dtype != q_out.dtype:
                raise KernelError("cache and activations differ in dtype")
            if tuple(k_cache.shape[1:]) != (n_kv, page_size, head_dim) or tuple(v_cache.shape[1:]) != (n_kv, head_dim, page_size):
                raise KernelError(f"cache pages have shapes {tuple(k_cache.shape)}, {tuple(v_cache.shape)}")
        self._check(
            self.lib.yk_rope_append(
                src.data_ptr(), _code(src.dtype), n_splits, round_sum, src_stride, q_out.data_ptr(), _code(q_out.dtype),
                q_out.stride(0), n, n_heads, n_kv, head_dim,
                positions.data_ptr(), _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None,
                rotary_dim, int(bool(interleaved)), max_pos,
                _ptr(k_cache) if n_kv else None, _ptr(v_cache) if n_kv else None,
                _ptr(slots) if n_kv else None, page_size, self._stream(),
            )
        )
        return q_out

    # ------------------------------------------------------------------ attention
    @staticmethod
    def attention_plan(column_groups: int, key_blocks: int) -> Tuple[int, int]:
        """(waves per workgroup, splits across workgroups) for the short-span kernel: the
        keys of a column group are divided until the launch has about ATTN_TARGET_WAVES
        waves, first among the waves of a workgroup (merged through LDS, no second kernel),
        then across workgroups (merged by the combine kernel)."""
        par = max(1, min(-(-ATTN_TARGET_WAVES // max(1, column_groups)), key_blocks))
        if par == 1:
            return 1, 1
        return 4, max(1, min(-(-par // 4), 256))

    @staticmethod
    def attention_long_splits(workgroups: int, key_blocks: int, col_tiles: int = 1) -> int:
        """Splits of the keys for the long-span kernel: one where the tiles alone fill the GPU
        (a prompt of a few thousand tokens); more where few tiles meet a long context (a
        portion of a prompt whose earlier portions are cached): as many as still leave all
        workgroups on the GPU at once (three a compute unit with one column tile a wave, two
        with two; a second, partly filled round costs more than the finer split gains: a
        480-token portion against 3,616 cached, one column tile, 3 / 4 / 5 splits 71.8 / 76.4 /
        73.3 us; two column tiles, 3 / 4 / 5 splits 74.3 / 64.5 / 76.9), at least 8 key blocks
        a split."""
        slots = 768 if col_tiles == 1 else 512
        return max(1, min(slots // max(1, workgroups), key_blocks // 8, 16))

    @staticmethod
    def rope_in_launch(rotation, append: bool) -> "RopeInLaunch":
        """What ``attention(rope=)`` takes, from a position encoding's ``Rotation`` (None: no
        rotation, the launch only appends) and whether the projection's rows hold keys and
        values to append."""
        if rotation is None:
            return RopeInLaunch(None, None, 0, False, append)
        return RopeInLaunch(rotation.cos, rotation.sin, rotation.rotary_dim, rotation.interleaved, append)

    def attention_can_rotate(self, act_dtype: torch.dtype, head_dim: int) -> bool:
        """Whether ``attention`` takes ``rope=`` for such a mixer: the matrix-core kernel for
        short spans can rotate queries and append keys and values itself."""
        return act_dtype == torch.bfloat16 and bool(self._ask("yk_attn_mfma_supported", head_dim))

    def attention(self, qkv, n_heads, n_kv, head_dim, k_cache, v_cache, page_size,
                  scale, window, ctx, group, tiles, long_tiles=None, plan=None, long_plan=None,
                  long_col_tiles: int = 1, token_cols=None, rope: Optional["RopeInLaunch"] = None):
        """Queries are the first n_heads heads of each row of ``qkv`` (whatever follows
        them in the row is skipped); keys and values come from the cache through the
        block table of ``group``.  ``long_tiles`` hold up to
        ``attention_long_span_tile(n_heads, n_kv, long_col_tiles)`` tokens each.  ``plan``
        overrides ``attention_plan`` and ``long_plan`` ``attention_long_splits`` (tests,
        measurements).  With ``token_cols`` (``attention_token_columns`` of the same short
        tiles) the caller takes a ``SplitAttention`` as well: what a step of up to 16 tokens,
        none of them in a long tile, leaves when its keys were split across workgroups.

        ``rope`` (only where ``attention_can_rotate``, and only for steps whose spans are single
        tokens): ``qkv`` is then the projection's raw output (a tensor or a ``SplitSum``) and
        the launch does what ``rope_append`` would have done before it: it rotates the queries
        and, with ``rope.append``, rotates the tokens' keys, uses them and their values, and
        stores both in the pages."""
        if rope is not None:
            return self._attention_rope(qkv, n_heads, n_kv, head_dim, k_cache, v_cache, page_size, scale, window,
                                        ctx, group, tiles, plan, token_cols, rope)
        self._rows(qkv, "qkv")
        n = qkv.shape[0]
        bt = ctx.arrays[f"block_table_g{group}"]
        if tuple(k_cache.shape[1:]) != (n_kv, page_size, head_dim) or tuple(v_cache.shape[1:]) != (n_kv, head_dim, page_size):
            raise KernelError(f"cache pages have shapes {tuple(k_cache.shape)}, {tuple(v_cache.shape)}")
        if k_cache.dtype != qkv.dtype:
            raise KernelError("cache and activations differ in dtype")
        out = torch.empty((n, n_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
        use_mfma = (
            qkv.dtype == torch.bfloat16
            and self._ask("yk_attn_mfma_supported", head_dim)
            and qkv.stride(0) % 8 == 0
            and qkv.data_ptr() % 16 == 0
        )
        if use_mfma and long_tiles is not None and long_tiles.shape[0] > 0:
            n_long = long_tiles.shape[0]
            hpt = self._ask("yk_attn_heads_per_tile", n_heads, n_kv)
            groups = n_long * n_kv * (-(-(n_heads // n_kv) // hpt))
            long_splits = long_plan if long_plan is not None else self.attention_long_splits(groups, max(1, -(-ctx.max_ctx // 64)), int(long_col_tiles))
            ws_floats = self._ask("yk_attn_mfma_workspace", 4 * long_col_tiles * n_long, n_heads, n_kv, head_dim, long_splits)
            ws = self._ws(ws_floats) if ws_floats else None
            self._check(
                self.lib.yk_attn_mfma_prefill(
                    qkv.data_ptr(), qkv.stride(0), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                    long_tiles.data_ptr(), n_long, bt.data_ptr(), bt.shape[1], page_size, head_dim,
                    n_heads, n_kv, float(scale), int(window), long_splits, int(long_col_tiles), _ptr(ws),
                    0 if ws is None else ws.numel(), int(self.long_span_pages_in_lds),
                    self._stream(),
                )
            )
        if use_mfma and tiles.shape[0] == 0:
            return out
        if use_mfma:
            n_tiles = tiles.shape[0]
            hpt = self._ask("yk_attn_heads_per_tile", n_heads, n_kv)
            chunks = -(-(n_heads // n_kv) // hpt)
            key_blocks = max(1, -(-ctx.max_ctx // 64))
            waves, splits = plan or self.attention_plan(n_tiles * n_kv * chunks, key_blocks)
            ws_floats = self._ask("yk_attn_mfma_workspace", n_tiles, n_heads, n_kv, head_dim, splits)
            ws = self._ws(ws_floats) if ws_floats else None
            leave = bool(token_cols is not None and splits > 1 and n <= MERGE_IN_PRODUCT_MAX_TOKENS and (long_tiles is None or long_tiles.shape[0] == 0))
            self._check(
                self.lib.yk_attn_mfma(
                    qkv.data_ptr(), qkv.stride(0), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                    tiles.data_ptr(), n_tiles, bt.data_ptr(), bt.shape[1], page_size, head_dim, n_heads, n_kv,
                    float(scale), int(window), waves, splits, _ptr(ws), 0 if ws is None else ws.numel(), int(leave),
                    self._stream(),
                )
            )
            if leave:
                return SplitAttention(self, ws, tiles, token_cols, n, n_heads, n_kv, head_dim, splits)
        else:
            self._check(
                self.lib.yk_attn_generic(
                    qkv.data_ptr(), qkv.stride(0), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                    _code(qkv.dtype), ctx.arrays["positions"].data_ptr(), ctx.arrays["token_seq"].data_ptr(),
                    bt.data_ptr(), bt.shape[1], n, page_size, head_dim, n_heads, n_kv, float(scale), int(window),
                    self._stream(),
                )
            )
        return out

    def _attention_rope(self, qkv, n_heads, n_kv, head_dim, k_cache, v_cache, page_size, scale, window,
                        ctx, group, tiles, plan, token_cols, rope: "RopeInLaunch"):
        n_splits_src, round_sum, src = 1, 0, qkv
        if isinstance(qkv, SplitSum):
            qkv.check_live()
            n_splits_src, round_sum, src = qkv.n_splits, qkv.round_sum, qkv.tensor
            n, cols = qkv.shape
            src_stride = cols
        else:
            self._rows(qkv, "qkv")
            n, cols = qkv.shape
            src_stride = qkv.stride(0)
        if ctx.max_qlen != 1 or tiles.shape[0] != n:
            raise KernelError("attention with rotary inside takes steps of single tokens only")
        if not self.attention_can_rotate(k_cache.dtype, head_dim):
            raise KernelError("attention with rotary inside needs bfloat16 pages and a head size of 64 or 128")
        if cols != (n_heads + (2 * n_kv if rope.append else 0)) * head_dim:
            raise KernelError(f"projection rows have {cols} elements, expected {(n_heads + (2 * n_kv if rope.append else 0)) * head_dim}")
        if tuple(k_cache.shape[1:]) != (n_kv, page_size, head_dim) or tuple(v_cache.shape[1:]) != (n_kv, head_dim, page_size):
            raise KernelError(f"cache pages have shapes {tuple(k_cache.shape)}, {tuple(v_cache.shape)}")
        max_pos = 0
        if rope.rotary_dim:
            cos, sin = rope.cos, rope.sin
            if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rope.rotary_dim // 2:
                raise KernelError("rotary tables must be float32 [positions, rotary_dim/2]")
            max_pos = cos.shape[0]
        bt = ctx.arrays[f"block_table_g{group}"]
        out = torch.empty((n, n_heads * head_dim), dtype=torch.bfloat16, device=src.device)
        hpt = self._ask("yk_attn_heads_per_tile", n_heads, n_kv)
        chunks = -(-(n_heads // n_kv) // hpt)
        key_blocks = max(1, -(-ctx.max_ctx // 64))
        waves, splits = plan or self.attention_plan(n * n_kv * chunks, key_blocks)
        ws_floats = self._ask("yk_attn_mfma_workspace", n, n_heads, n_kv, head_dim, splits)
        ws = self._ws(ws_floats) if ws_floats else None
        leave = bool(token_cols is not None and splits > 1 and n <= MERGE_IN_PRODUCT_MAX_TOKENS)
        self._check(
            self.lib.yk_attn_mfma_rope(
                src.data_ptr(), _code(src.dtype), n_splits_src, round_sum, src_stride, n,
                _ptr(rope.cos) if rope.rotary_dim else None, _ptr(rope.sin) if rope.rotary_dim else None,
                int(rope.rotary_dim), int(bool(rope.interleaved)), max_pos, int(bool(rope.append)),
                out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), tiles.data_ptr(), n, bt.data_ptr(), bt.shape[1],
                page_size, head_dim, n_heads, n_kv, float(scale), int(window), waves, splits, _ptr(ws),
                0 if ws is None else ws.numel(), int(leave), self._stream(),
            )
        )
        if leave:
            return SplitAttention(self, ws, tiles, token_cols, n, n_heads, n_kv, head_dim, splits)
        return out

    # ----------------------------------------------------------------- activation
    def gated_act(self, gu, activation: str, out_dtype: Optional[torch.dtype] = None, group: int = 0) -> torch.Tensor:
        """act(gate) * up for gate/up columns [gate | up] (group 0) or alternating in groups
        of ``group`` columns (see ``pack_gate_up``)."""
        n_splits, round_sum = 1, 0
        src = gu
        if isinstance(gu, SplitSum):
            gu.check_live()
            n_splits, round_sum, src = gu.n_splits, gu.round_sum, gu.tensor
            rows, cols = gu.shape
            out_dtype = out_dtype or torch.bfloat16
        else:
            self._rows(gu, "gate/up")
            if not gu.is_contiguous():
                raise KernelError("gate/up must be contiguous")
            rows, cols = gu.shape
            out_dtype = out_dtype or gu.dtype
        if cols % 2:
            raise KernelError("gate/up must have an even number of columns")
        act = {"silu": 0, "gelu_tanh": 1}.get(activation)
        if act is None:
            raise KernelError(f"unknown activation {activation!r}")
        inter = cols // 2
        out = torch.empty((rows, inter), dtype=out_dtype, device=src.device)
        self._check(
            self.lib.yk_gated_act(src.data_ptr(), _code(src.dtype), n_splits, round_sum, out.data_ptr(), _code(out_dtype),
                                  rows, inter, act, int(group), self._stream())
        )
        return out

    # ------------------------------------------------------------------- sampling
    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        if logits.dtype != torch.float32 or not logits.is_contiguous() or logits.dim() != 2:
            raise KernelError("argmax takes contiguous float32 logits [rows, vocab]")
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        ws = self._ws(64 * logits.shape[0])
        lib = self._library("sampling")
        self._check(lib.yk_argmax(logits.data_ptr(), out.data_ptr(), logits.shape[0], logits.shape[1],
                                  ws.data_ptr(), ws.numel(), self._stream()), lib)
        return out

    def sample(self, logits, temperature, top_k, top_p, seeds, draws, whole_row: bool = False, paths=None) -> torch.Tensor:
        """Per row: temperature (float32; 0 = greedy), top_k (int32; 0 = off), top_p
        (float32), seed and draw number (int32).  Returns int32 token ids.  Rows of a large
        vocabulary are divided among workgroups; ``whole_row`` forces one workgroup a row on
        the path that never narrows the row down to candidates (for tests), and ``paths``
        (int32, one per row) receives which way each divided row went: 0 greedy, 1 a race
        over the row, 3 settled among candidates, 4 left to one workgroup after all."""
        if logits.dtype != torch.float32 or not logits.is_contiguous() or logits.dim() != 2:
            raise KernelError("sample takes contiguous float32 logits [rows, vocab]")
        rows = logits.shape[0]
        for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                            ("top_p", top_p, torch.float32), ("seeds", seeds, torch.int32), ("draws", draws, torch.int32)):
            if t.dtype != dt or t.numel() != rows or not t.is_contiguous():
                raise KernelError(f"sample: {name} must be {dt} with one entry per row")
        if paths is not None and (paths.dtype != torch.int32 or paths.numel() != rows or not paths.is_contiguous()):
            raise KernelError("sample: paths must be int32 with one entry per row")
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        lib = self._library("sampling")
        need = 0 if whole_row else int(lib.yk_sample_workspace_bytes(rows, logits.shape[1]))
        ws = self._ws((need + 3) // 4) if need else None
        self._check(
            lib.yk_sample(
                logits.data_ptr(), out.data_ptr(), rows, logits.shape[1], temperature.data_ptr(), top_k.data_ptr(),
                top_p.data_ptr(), seeds.data_ptr(), draws.data_ptr(), int(bool(whole_row)),
                _ptr(ws), 0 if ws is None else ws.numel() * 4, _ptr(paths), self._stream(),
            ),
            lib,
        )
        return out

    def cache_tiled(self, dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
        """Whether pages of this kind are kept in the order the matrix-core attention loads
        them rather than as plain [slot, dim] keys and [dim, slot] values.  The kernels that
        write and read pages decide alike from the same three numbers; code that fills or
        inspects pages by hand (tests) has to ask."""
        return bool(self.lib.yk_cache_tiled(_code(dtype), int(head_dim), int(page_size)))

    # ------------------------------------------------------------------ machine probes
    def probe_stream_read(self, data: torch.Tensor, workgroups: int, sink: torch.Tensor, nontemporal: bool = False) -> None:
        """Reads every byte of ``data`` once with a plain streaming kernel (for timing);
        ``nontemporal`` marks the loads as not to be kept in the caches."""
        lib = self._library("probe")
        self._check(lib.yk_probe_stream_read(data.data_ptr(), data.numel() * data.element_size(), int(workgroups),
                                             int(bool(nontemporal)), sink.data_ptr(), self._stream()), lib)

    def probe_mfma_bf16(self, workgroups: int, iterations: int, sink: torch.Tensor) -> int:
        """Issues a loop of bfloat16 matrix-core instructions from registers; returns its flop count."""
        lib = self._library("probe")
        self._check(lib.yk_probe_mfma_bf16(int(workgroups), int(iterations), sink.data_ptr(), self._stream()), lib)
        return int(workgroups) * 4 * int(iterations) * 4 * 16384
