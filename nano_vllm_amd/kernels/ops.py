"""The operations the parts call, bound to the HIP kernels under csrc/.

Each method checks on the host that operand shapes, strides and types match what its
kernel and grid assume, then launches on torch's current stream.  torch is the allocator
and stream owner; the only library computation left is the bfloat16 matrix product for
many rows, where the reference uses a library as well (nanovllm/layers/linear.py:51,73,153).

Cache layouts (chosen for the attention kernels):
    K [pages, kv_heads, page_size, head_dim]
    V [pages, kv_heads, page_size / vt, head_dim, vt]   transposed (keys of a channel are contiguous)
                                                        in tiles of vt = v_tile(page_size) keys
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import library
from .library import KernelError

_SUFFIX = {torch.bfloat16: "bf16", torch.float32: "f32"}

c_i32, c_i64, c_f32, c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


def v_tile(page_size: int) -> int:
    """Keys per tile of the V cache: 32 when the page size is a multiple of 32, else the page."""
    return 32 if page_size % 32 == 0 else page_size


def v_cache_shape(pages: int, kv_heads: int, head_dim: int, page_size: int):
    vt = v_tile(page_size)
    return (pages, kv_heads, page_size // vt, head_dim, vt)


def _p(t: Optional[torch.Tensor]):
    return None if t is None else c_ptr(t.data_ptr())


def _suffix(t: torch.Tensor) -> str:
    try:
        return _SUFFIX[t.dtype]
    except KeyError:
        raise KernelError(f"no kernels for element type {t.dtype}; bfloat16 and float32 are built") from None


def _rows2d(t: torch.Tensor, what: str) -> Tuple[int, int, int]:
    """(rows, width, row stride) of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what}: expected a 2-D tensor with contiguous rows, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")
    return t.shape[0], t.shape[1], t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, n: int, what: str):
    if t.dtype != torch.int32 or t.dim() != 1 or t.shape[0] != n or not t.is_contiguous():
        raise KernelError(f"{what}: expected contiguous int32[{n}], got {t.dtype}{tuple(t.shape)}")


class SplitSum:
    """A bfloat16 product left as float partial sums [splits, rows, width] (+ bias) by the
    weight-streaming kernel, for the next kernel to add up while it reads them: the norms and
    the q/k preparation take it in place of a tensor; anything else gets `tensor()`."""

    def __init__(self, kernels, sums: torch.Tensor, splits: int, rows: int, width: int, bias):
        self.kernels, self.sums, self.splits, self.rows, self.width, self.bias = kernels, sums, splits, rows, width, bias
        self.dtype = torch.bfloat16
        self.device = sums.device
        self.shape = (rows, width)
        self._tensor = None

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            out = torch.empty(self.shape, dtype=self.dtype, device=self.device)
            library.call("gemm_skinny", "bf16", "nva_linear_skinny_finish", _p(self.sums), c_i32(self.splits),
                         _p(self.bias), _p(out), c_i64(self.width), c_i32(0), c_i32(0), c_i64(self.rows),
                         c_i64(self.width), self.kernels._stream())
            self._tensor = out
        return self._tensor


class PendingProduct:
    """A bfloat16 product of many rows that the library has not run yet: x and the weight.  The
    norm that adds it to the residual stream runs it as residual <- residual + x @ weight.T, the sum
    in the product's own epilogue (float, rounded once), which saves a pass over the product;
    anything else gets `tensor()`, the plain product."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor):
        self.x, self.weight = x, weight
        self.dtype = x.dtype
        self.device = x.device
        self.shape = (x.shape[0], weight.shape[0])
        self._tensor = None

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = torch.nn.functional.linear(self.x, self.weight)
        return self._tensor

    def add_to(self, residual: torch.Tensor) -> torch.Tensor:
        return residual.addmm_(self.x, self.weight.t())


def _t(x):
    return x.tensor() if isinstance(x, (SplitSum, PendingProduct)) else x


def check_positions_fit(table: torch.Tensor, head_dim: int, max_position: Optional[int]) -> None:
    """The rotary kernels read row positions[t] of the table without a check on the device: a
    step whose positions are not all rows of the table is refused here.  The table's width is the
    number of channels that are rotated: the head's, or fewer (the first of the head)."""
    if (table.dtype != torch.float32 or table.dim() != 2 or not table.is_contiguous() or table.shape[1] % 2
            or not 0 < table.shape[1] <= head_dim):
        raise KernelError(f"rotary table must be float32 [positions, rot], rot even and at most the head's {head_dim}")
    if max_position is None:
        raise KernelError("rotation by a table needs max_position, the bound of the step's positions")
    if max_position > table.shape[0]:
        raise KernelError(f"a position of {max_position - 1} has no row in the rotary table of {table.shape[0]} "
                          f"positions (max_position_embeddings)")


MEDIUM_KERNEL_ROWS = 256    # rows of x that nva_linear_medium takes
TILE_KERNEL_ROWS = 256      # rows of x up to which the LDS-tiled product streams a weight (one tile of rows)
PREFILL_ROWS = 32       # query rows of one workgroup of the prefill attention kernel
PREFILL_MAX_TABLE = 4096    # pages of a block-table row the prefill attention kernel stages in LDS
GENERAL_TILED_MAX_HEAD_DIM = 128    # head sizes of nva_paged_attention_tiled


def retention_blocks(q_lens, first_seq: int):
    """How the retention kernel on the matrix cores cuts the step's portions (the requests from
    `first_seq` on) into blocks that run side by side: (tokens of a block, units, chains) with units a
    flat list of (request counted from first_seq, first token of the block within the portion, its
    tokens, blocks of the portion) and chains one of (first unit, blocks, request, tokens of the last
    block) for every portion of more than one block.  Blocks of 64 tokens, of more where that still
    leaves 64 blocks."""
    total = sum(q_lens[first_seq:])
    bt = 64
    while bt < 512 and total // bt > 64:
        bt *= 2
    units, chains = [], []
    for s in range(first_seq, len(q_lens)):
        n = q_lens[s]
        nb = (n + bt - 1) // bt
        if nb > 1:
            chains += [len(units) // 4, nb, s - first_seq, n - (nb - 1) * bt]
        for b in range(nb):
            units += [s - first_seq, b * bt, min(bt, n - b * bt), nb]
    return bt, units, chains


def state_space_blocks(q_lens, first_seq: int):
    """As retention_blocks, for the state-space layer's blocks as products: blocks of 64 tokens, which that kernel takes, as long
    as the step's portions hold at most 16384 tokens (a block's end state is kept until the pass over the blocks);
    beyond that the blocks double as retention's do."""
    total = sum(q_lens[first_seq:])
    if total > 16384:
        return retention_blocks(q_lens, first_seq)
    bt = 64
    units, chains = [], []
    for s in range(first_seq, len(q_lens)):
        n = q_lens[s]
        nb = (n + bt - 1) // bt
        if nb > 1:
            chains += [len(units) // 4, nb, s - first_seq, n - (nb - 1) * bt]
        for b in range(nb):
            units += [s - first_seq, b * bt, min(bt, n - b * bt), nb]
    return bt, units, chains


def prefill_tile_order(q_lens, starts, first_seq: int) -> list:
    """Flat [(request, row tile), ...] of the requests from `first_seq` on, from the tile that
    sees the most keys to the one that sees the fewest: the prefill attention kernel hands its
    workgroups out in this order, so that the long ones start first."""
    units = []
    for s in range(first_seq, len(q_lens)):
        n = q_lens[s]
        for t in range((n + PREFILL_ROWS - 1) // PREFILL_ROWS):
            units.append((starts[s] + min(n, (t + 1) * PREFILL_ROWS), s, t))
    units.sort(key=lambda u: (-u[0], u[1], u[2]))
    return [v for u in units for v in (u[1], u[2])]


# What choose_products measured, per device name: {(n, k, gated): {ceil(rows / 16): "library" | "medium" | "tile"}}.
# One table per process and device, shared by every HipKernels there, and kept in a file beside the
# compiled libraries, so that engines on the same model dispatch alike from one process to the next
# (the two kernels round their sums differently).
_product_choices: dict = {}


def _choice_file(write: bool = False) -> Optional[str]:
    """The record of the measured choices: named after the build of the product kernels it was
    measured with, in the first folder for compiled libraries that holds one (write: that can take one)."""
    import os
    from . import build
    lib = build.find_library("gemm_skinny", "bf16")
    tag = os.path.basename(lib).split(".")[1] if lib else "unbuilt"
    name = f"product_choice.{tag}.json"
    for d in build.build_dirs():
        path = os.path.join(d, name)
        if os.path.isfile(path) or (write and build._writable(d)):
            return path
    return None


def recorded_product_choices(device_name: str) -> dict:
    table = _product_choices.get(device_name)
    if table is None:
        import json
        table = _product_choices[device_name] = {}
        path = _choice_file()
        if path:
            try:
                with open(path) as f:
                    stored = json.load(f).get(device_name, {})
                for key, rows in stored.items():
                    n, k, gated = key.split(",")
                    table[(int(n), int(k), gated == "1")] = {int(r): c for r, c in rows.items()
                                                            if c in ("library", "medium", "tile")}
            except (OSError, ValueError, AttributeError):
                table.clear()                   # an unreadable record is measured again
    return table


def _write_product_choices() -> None:
    import json
    import os
    path = _choice_file(write=True)
    if not path:
        return
    stored = {dev: {f"{n},{k},{int(g)}": {str(r): c for r, c in sorted(rows.items())} for (n, k, g), rows in table.items()}
              for dev, table in _product_choices.items()}
    tmp = f"{path}.{os.getpid()}.tmp"
    try:
        with open(tmp, "w") as f:
            json.dump(stored, f, indent=1, sort_keys=True)
        os.replace(tmp, path)
    except OSError:
        pass                                    # the record is a convenience: without it the next process measures again


class HipKernels:
    """Every device operation of the engine.  Needs a GPU and the compiled libraries."""

    name = "hip"
    max_burst_groups = 4        # cache groups nva_advance_decode takes in one launch

    def __init__(self, device="cuda:0", dtype: torch.dtype = torch.bfloat16, quiet: bool = False, modules=None):
        """modules: the kernel modules to compile and load now (None: all of the element type);
        whatever else is called later is compiled then."""
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine runs on HIP kernels only and has no CPU path")
        if dtype not in _SUFFIX:
            raise KernelError(f"no kernels for element type {dtype}; bfloat16 and float32 are built")
        self.device = torch.device(device)
        self.dtype = dtype
        self.suffix = _SUFFIX[dtype]
        library.preload(self.suffix, quiet=quiet, modules=modules)       # compiles what this element type needs
        # bit 0: a token id outside the vocabulary; bit 1: a visible key without a page;
        # bit 2: the decode attention's plan outgrew its bound
        self.fault_flag = torch.zeros(1, dtype=torch.int32, device=self.device)
        # Rows up to which the bfloat16 product runs on the engine's own kernels.
        props = torch.cuda.get_device_properties(self.device)
        cus = props.multi_processor_count
        self.cus = cus
        self.own_matmul_rows = 16           # bfloat16 products with more rows go to the library ...
        self.skinny_max_rows = 64           # ... unless the weight is small (see _own_rows); the kernel's limit
        self.small_weight_bytes = 64 << 20
        self.medium_max_rows = 224          # rows of x the kernel for medium row counts is used for (it takes 256)
        self.medium_row_tiles = 2           # 1: one block of 16 weight rows per wave in the kernel for up to 256 rows (tests)
        self.medium_shape = None            # (waves, row tiles, ranges of k) forced on that kernel (tests)
        self.medium_target_workgroups = cus  # one workgroup per CU
        self.team_max_rows = 16             # rows of x of the kernel whose waves split k inside a workgroup, for wide weights
        # A weight is wide when every CU's team gets two blocks of 16 rows at least: with one block a
        # team loads its x for that block alone and keeps nothing, and a weight with fewer blocks than
        # twice the CUs leaves CUs idle or unevenly loaded; such a weight is split over k instead.
        self.team_min_weight_rows = 2 * 16 * cus
        self.medium_max_weight_rows = self.team_min_weight_rows   # the widest weight the rule gives to the kernel for up to 256 rows
        self.teams = cus                    # one workgroup per CU
        self.skinny_waves_per_tile = 0      # waves of a workgroup that share rows of the weight and split k; 0: by rows of x
        # the k range of a few-row product is split until this many waves run: as many as the GPU
        # holds at four per SIMD (many short waves stream faster than few long ones)
        self.skinny_target_waves = 16 * cus
        # (n, k, gated) -> {ceil(rows / 16): "library" | "medium" | "tile"}: what choose_products measured on
        # this kind of device, in this process or an earlier one; where it has no entry the rules of
        # _own_kernel decide.  Every HipKernels of the process shares the table.
        self.product_choice = recorded_product_choices(props.name)
        self.choice_margin = 0.10           # the rule's kernel stays unless the other is faster by more than this
        self.tile_for_wide_weights = True   # False: the rule never names the LDS-tiled kernel (tests)
        self.tile_shape = None              # (shape, stages, ranges[, columns per workgroup]) forced on the LDS-tiled kernel (tests)
        self.tile_even_shares = True        # False: the LDS-tiled kernel's workgroups always take whole tiles (tests)
        self.fuse_split_sums = True         # False: every product is finished by its own pass
        # False: attention always runs the general kernel (tests compare the two)
        self.mfma_attention = True
        # False: retention always runs the general kernel
        self.mfma_retention = True
        # False: single tokens run the chunked kernels as chunks of one token
        self.retention_decode_kernel = True
        # False: a portion's chunks always run one after the other
        self.retention_blocks_side_by_side = True
        # False: the general kernel runs one wave per token for portions of prompts too (the same bits, slower)
        self.tiled_general_attention = True
        # False: the general kernel walks all of a token's keys in one workgroup, however many
        self.shared_general_attention = True
        # False: the state-space layer runs a portion's tokens one after the other, whatever its length
        self.state_space_blocks_side_by_side = True
        # how the recurrence holds a state of 65 to 128 rows: 0 two lanes a column (what serves), 1 a thread a column
        # with scalar operands, 2 four lanes a column, 3 the second pass of the blocks on the vector units, 4 single
        # tokens through the kernel of the portions, 6 blocks from a zero state as products on the matrix cores (measurements)
        self.state_space_shape = 0

    # ------------------------------------------------------------------ helpers
    def _stream(self):
        return c_ptr(torch.cuda.current_stream(self.device).cuda_stream)

    def check_faults(self) -> None:
        """Reads the device-side fault flags (a synchronising copy) and raises on any."""
        flags = int(self.fault_flag.item())
        if flags:
            self.fault_flag.zero_()
            what = []
            if flags & 1:
                what.append("a token id outside the vocabulary reached the embedding")
            if flags & 2:
                what.append("attention met a visible key whose page is missing from the block table")
            if flags & 4:
                what.append("the decode attention's plan needed more segments than it was sized for")
            if flags & ~7:
                what.append(f"unknown flags {flags & ~7:#x}")
            raise KernelError("device-side check failed: " + "; ".join(what))

    # ------------------------------------------------------------------ rows
    def embedding(self, table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out[t] = table[ids[t]]; also used to pick rows of activations."""
        rows, width, stride = _rows2d(table, "embedding table")
        n = ids.shape[0]
        _i32(ids, n, "embedding ids")
        if out is None:
            out = torch.empty((n, width), dtype=table.dtype, device=table.device)
        _, ow, ostride = _rows2d(out, "embedding out")
        if ow != width or out.dtype != table.dtype or out.shape[0] != n:
            raise KernelError("embedding: output does not match the table")
        library.call("embed", _suffix(table), "nva_gather_rows", _p(table), c_i64(stride), c_i64(rows), _p(ids),
                     _p(out), c_i64(ostride), c_i64(n), c_i32(width), _p(self.fault_flag), self._stream())
        return out

    gather_rows = embedding

    def embedding_scaled(self, table: torch.Tensor, ids: torch.Tensor, scale: float) -> torch.Tensor:
        """float32 out[t] = table[ids[t]] * scale: the start of a residual stream kept in float32."""
        rows, width, stride = _rows2d(table, "embedding table")
        n = ids.shape[0]
        _i32(ids, n, "embedding ids")
        out = torch.empty((n, width), dtype=torch.float32, device=table.device)
        library.call("embed", _suffix(table), "nva_gather_scale_rows", _p(table), c_i64(stride), c_i64(rows), _p(ids),
                     _p(out), c_i64(width), c_i64(n), c_i32(width), c_f32(float(scale)), _p(self.fault_flag), self._stream())
        return out

    # ------------------------------------------------------------------ norms
    def _norm_weight(self, weight: torch.Tensor, width: int, x: torch.Tensor):
        if weight.dim() != 1 or weight.shape[0] != width or not weight.is_contiguous():
            raise KernelError(f"norm weight must be contiguous [{width}], got {tuple(weight.shape)}")
        if weight.dtype == torch.float32:
            return 1
        if weight.dtype != x.dtype:
            raise KernelError(f"norm weight is {weight.dtype}; expected float32 or the input's {x.dtype}")
        return 0

    def _norm_of_partials(self, x: "SplitSum", residual, weight, eps, out):
        rows, width = x.shape
        wf = self._norm_weight(weight, width, x)
        rs = 0
        if residual is not None:
            rrows, rw, rs = _rows2d(residual, "add_rms_norm residual")
            if (rrows, rw) != (rows, width) or residual.dtype != x.dtype:
                raise KernelError("add_rms_norm: residual does not match the input")
        if out is None:
            out = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        orows, ow, os_ = _rows2d(out, "rms_norm output")
        if (orows, ow) != (rows, width) or out.dtype != x.dtype:
            raise KernelError("rms_norm: output does not match the input")
        library.call("norm", "bf16", "nva_rms_norm_of_partials", _p(x.sums), c_i32(x.splits), c_i64(rows * width),
                     _p(x.bias), _p(residual), c_i64(rs), _p(weight), c_i32(wf), _p(out), c_i64(os_), c_i64(rows),
                     c_i32(width), c_f32(eps), self._stream())
        return out

    def rms_norm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None):
        if isinstance(x, SplitSum):
            return self._norm_of_partials(x, None, weight, eps, out)
        x = _t(x)
        rows, width, xs = _rows2d(x, "rms_norm input")
        wf = self._norm_weight(weight, width, x)
        if out is None:
            out = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        orows, ow, os_ = _rows2d(out, "rms_norm output")
        if (orows, ow) != (rows, width) or out.dtype != x.dtype:
            raise KernelError("rms_norm: output does not match the input")
        library.call("norm", _suffix(x), "nva_rms_norm", _p(x), c_i64(xs), _p(weight), c_i32(wf), _p(out),
                     c_i64(os_), c_i64(rows), c_i32(width), c_f32(eps), self._stream())
        return out

    def add_rms_norm(self, x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                     out: Optional[torch.Tensor] = None):
        """residual <- x + residual (in place); returns (norm(residual) * weight, residual)."""
        if isinstance(x, SplitSum):
            return self._norm_of_partials(x, residual, weight, eps, out), residual
        if isinstance(x, PendingProduct):
            if (residual.dim() != 2 or tuple(residual.shape) != x.shape or residual.dtype != x.dtype
                    or residual.stride(1) != 1):
                raise KernelError("add_rms_norm: residual does not match the input")
            return self.rms_norm(x.add_to(residual), weight, eps, out=out), residual
        rows, width, xs = _rows2d(x, "add_rms_norm input")
        rrows, rw, rs = _rows2d(residual, "add_rms_norm residual")
        if (rrows, rw) != (rows, width) or residual.dtype != x.dtype:
            raise KernelError("add_rms_norm: residual does not match the input")
        wf = self._norm_weight(weight, width, x)
        if out is None:
            out = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        orows, ow, os_ = _rows2d(out, "add_rms_norm output")
        if (orows, ow) != (rows, width) or out.dtype != x.dtype:
            raise KernelError("add_rms_norm: output does not match the input")
        library.call("norm", _suffix(x), "nva_add_rms_norm", _p(x), c_i64(xs), _p(residual), c_i64(rs), _p(weight),
                     c_i32(wf), _p(out), c_i64(os_), c_i64(rows), c_i32(width), c_f32(eps), self._stream())
        return out, residual

    def stream_rms_norm(self, addends, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                        offset: float = 0.0, out: Optional[torch.Tensor] = None):
        """The norm of a residual stream that is kept in float32 whatever the element type:
        residual <- residual + sum(addends) in place (residual None: a new stream that starts as the
        sum of the addends), then y = residual * rsqrt(mean(residual^2) + eps) * (offset + weight),
        all in float and rounded once.  addends: up to two tensors of the element type [rows, width].
        Returns (y, residual)."""
        if any(hasattr(a, "mult") for a in addends):
            if len(addends) != 1 or residual is None or offset != 0.0:
                raise KernelError("stream_rms_norm: an addend with a norm of its own comes alone, into a stream that exists, "
                                  "and goes with a plain weight")
            return self._stream_post_norm(addends[0], residual, weight, eps, out)
        # a product left as partial sums is added up here, while it is read; anything else is a tensor
        addends = [a if isinstance(a, SplitSum) and self.fuse_split_sums else _t(a) for a in addends]
        if len(addends) > 2 or (residual is None and not addends):
            raise KernelError("stream_rms_norm: one or two addends (none only with a stream that exists)")
        ref = addends[0] if addends else None
        if ref is None:
            if out is None:
                raise KernelError("stream_rms_norm: without addends the output tensor says the element type")
            rows, width = residual.shape
        else:
            rows, width = ref.shape
        args = []
        for a in addends:
            if tuple(a.shape) != (rows, width) or a.dtype != ref.dtype:
                raise KernelError("stream_rms_norm: the addends differ in shape or type")
            if isinstance(a, SplitSum):
                args += [None, c_i64(0), _p(a.sums), c_i32(a.splits), c_i64(rows * width), _p(a.bias)]
            else:
                _, _, as_ = _rows2d(a, "stream_rms_norm addend")
                args += [_p(a), c_i64(as_), None, c_i32(0), c_i64(0), None]
        for _ in range(2 - len(addends)):
            args += [None, c_i64(0), None, c_i32(0), c_i64(0), None]
        first = residual is None
        device = ref.device if ref is not None else residual.device
        if first:
            residual = torch.empty((rows, width), dtype=torch.float32, device=device)
        rrows, rw, rs = _rows2d(residual, "stream_rms_norm residual")
        if (rrows, rw) != (rows, width) or residual.dtype != torch.float32:
            raise KernelError("stream_rms_norm: the residual stream must be float32 of the addends' shape")
        dtype = ref.dtype if ref is not None else out.dtype
        if out is None:
            out = torch.empty((rows, width), dtype=dtype, device=device)
        orows, ow, os_ = _rows2d(out, "stream_rms_norm output")
        if (orows, ow) != (rows, width) or out.dtype != dtype:
            raise KernelError("stream_rms_norm: output does not match")
        wf = self._norm_weight(weight, width, out)
        library.call("norm", _suffix(out), "nva_stream_rms_norm", *args, _p(residual), c_i64(rs), c_i32(1 if first else 0),
                     _p(weight), c_i32(wf), c_f32(offset), _p(out), c_i64(os_), c_i64(rows), c_i32(width), c_f32(eps),
                     self._stream())
        return out, residual

    def stream_scaled_norm(self, addends, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                           weight2: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                           out2: Optional[torch.Tensor] = None, dtype: Optional[torch.dtype] = None):
        """Two norms of one float32 stream, and addends that enter it through a vector each:
        residual <- residual + sum of scale_i * addend_i, in place (residual None: a new stream that starts as the
        one addend, which then has no scale); y = residual * rsqrt(mean(residual^2) + eps) * weight, and y2 the
        same with weight2 where that is given; all in float, each rounded once.  addends: up to two pairs
        (tensor of the element type or a split product, vector [width] or None).  dtype: the outputs' element
        type where neither an addend nor an output tensor says it.  Returns (y, y2 or None, residual)."""
        pairs = [(a if isinstance(a, SplitSum) and self.fuse_split_sums else _t(a), s) for a, s in addends]
        if len(pairs) > 2 or (residual is None and len(pairs) != 1):
            raise KernelError("stream_scaled_norm: one or two addends (none with a stream that exists, one to start it)")
        ref = pairs[0][0] if pairs else None
        rows, width = (ref.shape if ref is not None else residual.shape)
        elem = ref.dtype if ref is not None else out.dtype if out is not None else dtype
        if elem is None:
            raise KernelError("stream_scaled_norm: without addends the output tensor or dtype says the element type")
        device = ref.device if ref is not None else residual.device
        scale_f32 = None
        args = []
        for a, sc in pairs:
            if tuple(a.shape) != (rows, width) or a.dtype != elem:
                raise KernelError("stream_scaled_norm: the addends differ in shape or type")
            if sc is not None:
                f = self._norm_weight(sc, width, a)
                if scale_f32 not in (None, f):
                    raise KernelError("stream_scaled_norm: the two scale vectors differ in type")
                scale_f32 = f
            if isinstance(a, SplitSum):
                args += [None, c_i64(0), _p(a.sums), c_i32(a.splits), c_i64(rows * width), _p(a.bias), _p(sc)]
            else:
                _, _, as_ = _rows2d(a, "stream_scaled_norm addend")
                args += [_p(a), c_i64(as_), None, c_i32(0), c_i64(0), None, _p(sc)]
        for _ in range(2 - len(pairs)):
            args += [None, c_i64(0), None, c_i32(0), c_i64(0), None, None]
        first = residual is None
        if first:
            if pairs[0][1] is not None:
                raise KernelError("stream_scaled_norm: the addend that starts a stream has no scale")
            residual = torch.empty((rows, width), dtype=torch.float32, device=device)
        rrows, rw, rs = _rows2d(residual, "stream_scaled_norm residual")
        if (rrows, rw) != (rows, width) or residual.dtype != torch.float32:
            raise KernelError("stream_scaled_norm: the residual stream must be float32 of the addends' shape")
        if out is None:
            out = torch.empty((rows, width), dtype=elem, device=device)
        if weight2 is not None and out2 is None:
            out2 = torch.empty((rows, width), dtype=elem, device=device)
        for o in (out, out2):
            if o is not None and (tuple(o.shape) != (rows, width) or o.dtype != elem or not o.is_contiguous()):
                raise KernelError("stream_scaled_norm: an output does not match")
        wf = self._norm_weight(weight, width, out)
        if weight2 is not None and self._norm_weight(weight2, width, out) != wf:
            raise KernelError("stream_scaled_norm: the two weights differ in type")
        library.call("norm", _suffix(out), "nva_stream_scaled_norm", *args, c_i32(scale_f32 or 0), _p(residual), c_i64(rs),
                     c_i32(1 if first else 0), _p(weight), _p(weight2), c_i32(wf), _p(out),
                     _p(out2) if weight2 is not None else None, c_i64(width), c_i64(rows), c_i32(width), c_f32(eps),
                     self._stream())
        return out, (out2 if weight2 is not None else None), residual

    def _stream_post_norm(self, addend, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                          out: Optional[torch.Tensor] = None):
        """residual <- residual + mult * a / sqrt(mean(a^2) + eps_a) * w_a, then the stream's own norm, in one pass;
        `addend` carries a (elements, or a product left as partial sums), w_a, eps_a and mult."""
        a = addend.x if isinstance(addend.x, SplitSum) and self.fuse_split_sums else _t(addend.x)
        rows, width = a.shape
        rrows, rw, rs = _rows2d(residual, "stream_rms_norm residual")
        if (rrows, rw) != (rows, width) or residual.dtype != torch.float32:
            raise KernelError("stream_rms_norm: the residual stream must be float32 of the addend's shape")
        if out is None:
            out = torch.empty((rows, width), dtype=a.dtype, device=residual.device)
        orows, ow, os_ = _rows2d(out, "stream_rms_norm output")
        if (orows, ow) != (rows, width) or out.dtype != a.dtype:
            raise KernelError("stream_rms_norm: output does not match")
        wf = self._norm_weight(weight, width, out)
        awf = self._norm_weight(addend.weight, width, out)
        if isinstance(a, SplitSum):
            src = [None, c_i64(0), _p(a.sums), c_i32(a.splits), c_i64(rows * width), _p(a.bias)]
        else:
            _, _, as_ = _rows2d(a, "stream_rms_norm addend")
            src = [_p(a), c_i64(as_), None, c_i32(0), c_i64(0), None]
        library.call("norm", _suffix(out), "nva_stream_post_norm", *src, _p(addend.weight), c_i32(awf), c_f32(float(addend.eps)),
                     c_f32(float(addend.mult)), _p(residual), c_i64(rs), _p(weight), c_i32(wf), _p(out), c_i64(os_), c_i64(rows),
                     c_i32(width), c_f32(eps), self._stream())
        return out, residual

    def stream_dyt(self, addends, residual: Optional[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor,
                   alpha: torch.Tensor, out: Optional[torch.Tensor] = None):
        """The Dynamic Tanh norm of a residual stream kept in float32: residual <- residual + sum(addends) in
        place (residual None: a new stream that starts as the sum), then y = tanh(alpha * residual) * weight +
        bias, all float, rounded once.  addends: one or two tensors of the element type [rows, width]; weight
        and bias float32 [width], alpha a float32 tensor of one number (read on the device).  Returns
        (y, residual)."""
        addends = [_t(a) for a in addends]
        if not 1 <= len(addends) <= 2:
            raise KernelError("stream_dyt: one or two addends")
        ref = addends[0]
        rows, width = ref.shape
        args = []
        for a in addends:
            if tuple(a.shape) != (rows, width) or a.dtype != ref.dtype:
                raise KernelError("stream_dyt: the addends differ in shape or type")
            _, _, as_ = _rows2d(a, "stream_dyt addend")
            args += [_p(a), c_i64(as_)]
        if len(addends) == 1:
            args += [None, c_i64(0)]
        first = residual is None
        if first:
            residual = torch.empty((rows, width), dtype=torch.float32, device=ref.device)
        rrows, rw, rs = _rows2d(residual, "stream_dyt residual")
        if (rrows, rw) != (rows, width) or residual.dtype != torch.float32:
            raise KernelError("stream_dyt: the residual stream must be float32 of the addends' shape")
        for v, what in ((weight, "weight"), (bias, "bias")):
            if v.dtype != torch.float32 or tuple(v.shape) != (width,) or not v.is_contiguous():
                raise KernelError(f"stream_dyt: {what} must be contiguous float32 [{width}]")
        if alpha.dtype != torch.float32 or alpha.numel() != 1:
            raise KernelError("stream_dyt: alpha must be one float32 number")
        if out is None:
            out = torch.empty((rows, width), dtype=ref.dtype, device=ref.device)
        orows, ow, os_ = _rows2d(out, "stream_dyt output")
        if (orows, ow) != (rows, width) or out.dtype != ref.dtype:
            raise KernelError("stream_dyt: output does not match")
        library.call("norm", _suffix(out), "nva_stream_dyt", *args, _p(residual), c_i64(rs), c_i32(1 if first else 0),
                     _p(weight), _p(bias), _p(alpha), _p(out), c_i64(os_), c_i64(rows), c_i32(width), self._stream())
        return out, residual

    def pair_norm_mean(self, a, wa: torch.Tensor, b, wb: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None):
        """(a * rsqrt(mean(a^2) + eps) * wa + b * rsqrt(mean(b^2) + eps) * wb) / 2 over rows of the model width;
        wa, wb float32 [width].  An input left as a split product's partial sums is added up while it is read."""
        a, b = [x if isinstance(x, SplitSum) and self.fuse_split_sums else _t(x) for x in (a, b)]
        rows, width = a.shape
        if tuple(b.shape) != (rows, width) or a.dtype != b.dtype:
            raise KernelError("pair_norm_mean: the inputs differ in shape or type")
        for w in (wa, wb):
            if w.dtype != torch.float32 or tuple(w.shape) != (width,) or not w.is_contiguous():
                raise KernelError(f"pair_norm_mean: the weights must be contiguous float32 [{width}]")
        args = []
        for x, w in ((a, wa), (b, wb)):
            if isinstance(x, SplitSum):
                args += [None, c_i64(0), _p(x.sums), c_i32(x.splits), c_i64(rows * width), _p(x.bias), _p(w)]
            else:
                _, _, xs = _rows2d(x, "pair_norm_mean input")
                args += [_p(x), c_i64(xs), None, c_i32(0), c_i64(0), None, _p(w)]
        if out is None:
            out = torch.empty((rows, width), dtype=a.dtype, device=a.device)
        orows, ow, os_ = _rows2d(out, "pair_norm_mean output")
        if (orows, ow) != (rows, width) or out.dtype != a.dtype:
            raise KernelError("pair_norm_mean: output does not match")
        library.call("norm", _suffix(out), "nva_pair_norm_mean", *args, _p(out), c_i64(os_), c_i64(rows), c_i32(width),
                     c_f32(eps), self._stream())
        return out

    def scale_(self, x: torch.Tensor, factor: float) -> torch.Tensor:
        """x <- x * factor in place; x float32 [rows, width]."""
        rows, width, xs = _rows2d(x, "scale_ input")
        if x.dtype != torch.float32:
            raise KernelError("scale_: the tensor must be float32")
        library.call("embed", self.suffix, "nva_scale_rows", _p(x), c_i64(xs), c_i64(rows), c_i32(width), c_f32(factor),
                     self._stream())
        return x

    # ------------------------------------------------------------------ feed-forward
    ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2}
    PLAIN_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2, "relu2": 3}

    def act(self, x: torch.Tensor, act: str = "relu2", out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """act(x), entry by entry: silu, relu, gelu_tanh or relu2 (the square of relu)."""
        if act not in self.PLAIN_ACTIVATIONS:
            raise KernelError(f"act: unknown activation {act!r}; known: {sorted(self.PLAIN_ACTIVATIONS)}")
        x = _t(x)
        rows, width, xs = _rows2d(x, "act input")
        if out is None:
            out = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        orows, ow, os_ = _rows2d(out, "act output")
        if (orows, ow) != (rows, width) or out.dtype != x.dtype:
            raise KernelError("act: output does not match the input")
        library.call("activation", _suffix(x), "nva_act", _p(x), c_i64(xs), _p(out), c_i64(os_), c_i64(rows), c_i32(width),
                     c_i32(self.PLAIN_ACTIVATIONS[act]), self._stream())
        return out

    # ------------------------------------------------------------------ routed feed-forward
    ROUTINGS = {"sigmoid_groups": 0, "softmax_top": 1, "softmax_choice": 2}

    def moe_route(self, logits: torch.Tensor, top: int, group_count: int, group_keep: int, scale: float,
                  routing: str = "sigmoid_groups", bias: Optional[torch.Tensor] = None):
        """From the router's float32 logits [tokens, experts]: int32 [tokens, top] experts and float32
        [tokens, top] weights (scale * sigmoid score).  Experts form group_count groups of neighbours; a
        group's score is the sum of its two largest scores; only experts of the group_keep best groups are
        chosen, the `top` with the largest scores.  routing "softmax_top": the `top` largest logits (plus the
        float32 bias [experts], if any) are chosen and weighted by the softmax over the chosen alone.  routing
        "softmax_choice": scores s = softmax(logits) over all experts; chosen by s + bias, within the group_keep groups
        whose largest s + bias is largest; weights s of the chosen over their sum (+ 1e-20).  logits may be the leading
        columns of wider rows."""
        rows, experts, ls = _rows2d(logits, "router logits")
        if logits.dtype != torch.float32:
            raise KernelError("moe_route: the logits must be float32")
        if routing not in self.ROUTINGS:
            raise KernelError(f"moe_route: unknown routing {routing!r}")
        if bias is not None and (bias.dtype != torch.float32 or tuple(bias.shape) != (experts,) or not bias.is_contiguous()):
            raise KernelError(f"moe_route: the bias must be contiguous float32 [{experts}]")
        ids = torch.empty((rows, top), dtype=torch.int32, device=logits.device)
        weights = torch.empty((rows, top), dtype=torch.float32, device=logits.device)
        library.call("moe", self.suffix, "nva_moe_route", _p(logits), c_i64(ls), c_i64(rows), c_i32(experts), c_i32(top),
                     c_i32(group_count), c_i32(group_keep), c_f32(scale), c_i32(self.ROUTINGS[routing]),
                     _p(bias), _p(ids), _p(weights), self._stream())
        return ids, weights

    def moe_experts(self, x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, up: torch.Tensor, down: torch.Tensor,
                    num_experts: int, act: str = "relu2", add=None, gated: bool = False,
                    add_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """y[t] = sum over the choices c of weights[t, c] * act(x[t] Wu_e^T) Wd_e^T with e = ids[t, c] (+ add[t]).
        up [E * ff, k] and down [E * k, ff] hold the experts' matrices one below the other.  gated: up is
        [E * 2 ff, k], an expert's gate rows and then its up rows, and the hidden layer act(x Wg_e^T) * (x Wu_e^T).
        An id from num_experts on is an identity: its output is x[t] itself.  add_gate, float32 [tokens] (a column of
        wider rows may be given): add[t] is multiplied by sigmoid(add_gate[t])."""
        if act not in self.PLAIN_ACTIVATIONS:
            raise KernelError(f"moe_experts: unknown activation {act!r}")
        x = _t(x)
        tokens, k, xs = _rows2d(x, "moe input")
        per = num_experts * (2 if gated else 1)
        if up.dim() != 2 or down.dim() != 2 or up.shape[0] % per or up.shape[1] != k or not up.is_contiguous() \
                or not down.is_contiguous() or up.dtype != x.dtype or down.dtype != x.dtype:
            raise KernelError("moe_experts: the experts' matrices do not fit the input")
        ff = up.shape[0] // per
        if tuple(down.shape) != (num_experts * k, ff):
            raise KernelError(f"moe_experts: down must be [{num_experts * k}, {ff}], got {tuple(down.shape)}")
        top = ids.shape[1] if ids.dim() == 2 else 0
        if ids.dtype != torch.int32 or tuple(ids.shape) != (tokens, top) or not ids.is_contiguous() or top <= 0 or \
                weights.dtype != torch.float32 or tuple(weights.shape) != (tokens, top) or not weights.is_contiguous():
            raise KernelError("moe_experts: ids int32 and weights float32, both contiguous [tokens, top]")
        add_stride = 0
        if add is not None:
            add = _t(add)
            arows, aw, add_stride = _rows2d(add, "moe addend")
            if (arows, aw) != (tokens, k) or add.dtype != x.dtype:
                raise KernelError("moe_experts: the addend does not match the input")
        gate_stride = 0
        if add_gate is not None:
            if add is None or add_gate.dtype != torch.float32 or add_gate.dim() != 1 or add_gate.shape[0] != tokens:
                raise KernelError("moe_experts: the addend's gate is float32 [tokens] and comes with an addend")
            gate_stride = add_gate.stride(0)
        pairs = tokens * top
        tile_rows = getattr(library.load("moe", self.suffix), f"nva_moe_tile_rows_{self.suffix}")
        bm = int(tile_rows(c_i64(pairs), c_i32(num_experts), c_i32(k), c_i32(ff)))
        max_tiles = pairs // bm + num_experts
        ints = torch.empty(2 * pairs + 3 * max_tiles + 1, dtype=torch.int32, device=x.device)
        hidden = torch.empty((pairs, ff), dtype=x.dtype, device=x.device)
        outs = torch.empty((pairs, k), dtype=x.dtype, device=x.device)
        y = torch.empty((tokens, k), dtype=x.dtype, device=x.device)
        library.call("moe", _suffix(x), "nva_moe_experts", _p(x), c_i64(xs), _p(ids), _p(weights), c_i64(tokens), c_i32(top),
                     c_i32(num_experts), c_i32(k), c_i32(ff), _p(up), _p(down), c_i32(self.PLAIN_ACTIVATIONS[act]),
                     c_i32(1 if gated else 0), _p(add), c_i64(add_stride), _p(add_gate), c_i64(gate_stride), _p(ints[:pairs]), _p(ints[pairs:2 * pairs]), _p(ints[2 * pairs:]), c_i64(max_tiles),
                     _p(hidden), _p(outs), _p(y), c_i64(k), self._stream())
        return y

    def act_mul(self, gate_up: torch.Tensor, act: str = "silu", out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """act(gate) * up of a row [gate | up]; act: silu, relu or gelu_tanh."""
        if act not in self.ACTIVATIONS:
            raise KernelError(f"act_mul: unknown activation {act!r}; known: {sorted(self.ACTIVATIONS)}")
        gate_up = _t(gate_up)
        rows, width, xs = _rows2d(gate_up, "act_mul input")
        if width % 2:
            raise KernelError("act_mul: the input holds gate and up halves, its width must be even")
        inner = width // 2
        if out is None:
            out = torch.empty((rows, inner), dtype=gate_up.dtype, device=gate_up.device)
        orows, ow, os_ = _rows2d(out, "act_mul output")
        if (orows, ow) != (rows, inner) or out.dtype != gate_up.dtype:
            raise KernelError("act_mul: output does not match the input")
        library.call("activation", _suffix(gate_up), "nva_act_mul", _p(gate_up), c_i64(xs), _p(out), c_i64(os_),
                     c_i64(rows), c_i32(inner), c_i32(self.ACTIVATIONS[act]), self._stream())
        return out

    def silu_mul(self, gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.act_mul(gate_up, "silu", out=out)

    # ------------------------------------------------------------------ matrix products
    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_float32: bool = False, out: Optional[torch.Tensor] = None, deferred: bool = False):
        """y = x @ weight.T (+ bias), weight [out, in].  float32 inputs run the engine's own
        float kernel; bfloat16 inputs with many rows run the library product (also for a float
        result of more than 16 rows), with few rows the weight-streaming kernels.  deferred: the caller hands the result to a norm or to the q/k
        preparation only, so a product split over k may come back as a SplitSum, and a library
        product as a PendingProduct."""
        x = _t(x)
        m, k, xs = _rows2d(x, "linear input")
        n, wk, ws = _rows2d(weight, "linear weight")
        if wk != k or weight.dtype != x.dtype:
            raise KernelError(f"linear: input [{m},{k}] {x.dtype} does not fit weight [{n},{wk}] {weight.dtype}")
        if bias is not None and (bias.shape != (n,) or bias.dtype != x.dtype or not bias.is_contiguous()):
            raise KernelError("linear: bias does not fit")
        out_dtype = torch.float32 if out_float32 else x.dtype
        if x.dtype == torch.bfloat16 and self._skinny_takes(x, xs, weight, ws, k):
            own = self._own_kernel(m, n, k)
            if own == "team":
                # a wide weight and few rows: k is split inside the workgroups, nothing is deferred
                if out is None:
                    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
                om, on, os_ = _rows2d(out, "linear output")
                if (om, on) != (m, n) or out.dtype != out_dtype:
                    raise KernelError("linear: output does not match")
                self._linear_team(x, xs, weight, ws, bias, out, os_, 1 if out_float32 else 0, m, n, k)
                return out
            if out_float32 and m > self.own_matmul_rows and own != "tile":
                # logits of many places: the library product with a float result reads the weight
                # once, where the streaming kernel would read it once per 64 rows
                y = torch.mm(x, weight.t(), out_dtype=torch.float32)
                if bias is not None:
                    y += bias.float()
                if out is not None:
                    om, on, _ = _rows2d(out, "linear output")
                    if (om, on) != (m, n) or out.dtype != out_dtype:
                        raise KernelError("linear: output does not match")
                    out.copy_(y)
                    return out
                return y
            if own == "tile" and not self._tile_takes(x, xs, weight, ws, m, n, k):
                own = None
            run = self._linear_medium if own == "medium" else self._linear_tile if own == "tile" else self._linear_skinny
            if deferred and own and not out_float32 and out is None and self.fuse_split_sums:
                return run(x, xs, weight, ws, bias, None, 0, False, False, m, n, k, defer=True)
            if own or out_float32:
                if out is None:
                    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
                om, on, os_ = _rows2d(out, "linear output")
                if (om, on) != (m, n) or out.dtype != out_dtype:
                    raise KernelError("linear: output does not match")
                if own in ("medium", "tile"):
                    run(x, xs, weight, ws, bias, out, os_, out_float32, False, m, n, k)
                    return out
                rows = self.skinny_max_rows      # more rows (logits of many places): that many at a time
                for r0 in range(0, m, rows):
                    r1 = min(m, r0 + rows)
                    self._linear_skinny(x[r0:r1], xs, weight, ws, bias, out[r0:r1], os_, out_float32, False, r1 - r0, n, k)
                return out
        if x.dtype == torch.bfloat16 and not out_float32:
            if deferred and bias is None and out is None and self.fuse_split_sums and xs == k and ws == k:
                return PendingProduct(x, weight)        # the library's product, run by whoever takes it
            y = torch.nn.functional.linear(x, weight, bias)
            if out is not None:
                out.copy_(y)
                return out
            return y
        if out is None:
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        om, on, os_ = _rows2d(out, "linear output")
        if (om, on) != (m, n) or out.dtype != out_dtype:
            raise KernelError("linear: output does not match")
        library.call("gemm", _suffix(x), "nva_linear_tiled", _p(x), c_i64(xs), _p(weight), c_i64(ws), _p(bias),
                     _p(out), c_i64(os_), c_i32(1 if out_dtype == torch.float32 and x.dtype != torch.float32 else 0),
                     c_i64(m), c_i64(n), c_i64(k), self._stream())
        return out

    def _own_kernel(self, m: int, n: int, k: int, gated: bool = False) -> Optional[str]:
        """Which of the engine's weight-streaming kernels takes a bfloat16 product of m rows with a
        weight [n, k]: "team", "skinny", "medium", "tile", or None for the library product.  Up to 16
        rows the engine's own kernels are as fast or faster for every weight ("team" for wide weights,
        whose waves split k inside a workgroup; "skinny" otherwise).  Beyond that the answer
        depends on the weight's shape and on what the library's heuristics pick for it, so it is
        measured once for the model's own weights (choose_products); without a measurement the
        rules of _rule_kernel stand: up to 224 rows the medium kernel for weights of few rows (the
        library has no split of k and leaves most of the GPU idle there), up to 256 rows the
        LDS-tiled kernel for wide ones (gate/up, the head), whose every workgroup takes all of k
        and does the gating itself; small wide weights whose k is no multiple of 64 stay with the
        skinny kernel up to 64 rows."""
        if m <= 0:
            return None
        if m <= self.team_max_rows and n >= self.team_min_weight_rows and k % 32 == 0:
            return "team"
        if m <= self.own_matmul_rows:
            return "skinny"
        measured = self.product_choice.get((n, k, gated))
        if measured is not None and (m + 15) // 16 in measured:
            choice = measured[(m + 15) // 16]
            return None if choice == "library" else choice
        return self._rule_kernel(m, n, k)

    def _rule_kernel(self, m: int, n: int, k: int) -> Optional[str]:
        """The unmeasured answer of _own_kernel beyond 16 rows."""
        if m <= self.medium_max_rows and n <= self.medium_max_weight_rows:
            return "medium"
        if m <= TILE_KERNEL_ROWS and k % 64 == 0 and n > self.medium_max_weight_rows and self.tile_for_wide_weights:
            return "tile"           # a wide weight (gate/up, the head): every workgroup takes all of k
        if m <= self.skinny_max_rows and 2 * n * k <= self.small_weight_bytes:
            return "skinny"
        return None

    def choose_products(self, tensors, max_rows: int, min_elements: int = 1 << 22, reps: int = 3,
                        remeasure: bool = False, record: bool = True) -> dict:
        """Measures, for every shape of weight among `tensors` (2-D bfloat16 of at least min_elements
        elements and at most 65536 rows: the layers' projections) and every row count that a captured
        decode step of up to max_rows requests can have beyond 16 (multiples of 16, at most 256),
        the library product against the engine's kernel for up to 256 rows, plain (as a norm or the
        q/k preparation consumes it) and with the SwiGLU gating, and keeps the faster per shape and
        row count in self.product_choice; the kernel that the rules of _own_kernel name stays unless
        the other is faster by more than choice_margin, so that two near-equal candidates do not
        swap from one measurement to the next.  The weights of one shape (one per layer) are used in
        turn, so that none is found in a cache.  What was measured before, in this process or in one
        that left its record beside the compiled libraries, is not measured again (remeasure: is),
        so engines on the same model dispatch alike; record=False leaves that file alone.  Returns
        the table."""
        import torch.nn.functional as F
        by_shape = {}
        for t in tensors:
            if t.dim() == 2 and t.dtype == torch.bfloat16 and t.is_cuda and t.numel() >= min_elements and \
                    t.shape[0] <= 65536 and t.is_contiguous():
                by_shape.setdefault(tuple(t.shape), []).append(t)
        rows = [m for m in range(32, min(max_rows, MEDIUM_KERNEL_ROWS) + 1, 16)]
        if not by_shape or not rows:
            return self.product_choice
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def timed(fn, weights) -> float:
            fn(weights[0])
            start.record()
            for i in range(reps):
                fn(weights[(i + 1) % len(weights)])
            stop.record()
            stop.synchronize()
            return start.elapsed_time(stop)

        measured = False
        for (n, k), weights in by_shape.items():
            if not self._skinny_takes(weights[0], k, weights[0], k, k):
                continue
            for gated in (False, True):
                if gated and n % 2:
                    continue
                table = {} if remeasure else dict(self.product_choice.get((n, k, gated), {}))
                for m in rows:
                    if m // 16 in table:
                        continue
                    x = torch.randn((m, k), dtype=torch.bfloat16, device=weights[0].device)
                    out = torch.empty((m, n // 2 if gated else n), dtype=torch.bfloat16, device=x.device)
                    cands = {}
                    if gated:
                        cands["library"] = lambda w: self.silu_mul(F.linear(x, w), out=out)
                        cands["medium"] = lambda w: self._linear_medium(x, k, w, k, None, out, n // 2, False, True, m, n, k)
                        if self._tile_takes(x, k, weights[0], k, m, n, k):
                            cands["tile"] = lambda w: self._linear_tile(x, k, w, k, None, out, n // 2, False, True, m, n, k)
                    else:
                        cands["library"] = lambda w: F.linear(x, w)
                        cands["medium"] = lambda w: self._linear_medium(x, k, w, k, None, None, 0, False, False, m, n, k, defer=True)
                        if self._tile_takes(x, k, weights[0], k, m, n, k):
                            cands["tile"] = lambda w: self._linear_tile(x, k, w, k, None, None, 0, False, False, m, n, k, defer=True)
                    # the smaller of two measurements each: a start-up has other work going on
                    times = {name: min(timed(fn, weights), timed(fn, weights)) for name, fn in cands.items()}
                    usual = self._rule_kernel(m, n, k)
                    usual = usual if usual in cands else "library"
                    best = min(times, key=times.get)
                    table[m // 16] = best if times[best] < (1.0 - self.choice_margin) * times[usual] else usual
                    measured = True
                self.product_choice[(n, k, gated)] = table
        if measured and record:
            _write_product_choices()
        return self.product_choice

    @staticmethod
    def _skinny_takes(x, xs, weight, ws, k) -> bool:
        return k % 8 == 0 and xs % 8 == 0 and ws % 8 == 0 and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0

    def _linear_skinny(self, x, xs, weight, ws, bias, out, os_, out_float32, swiglu, m, n, k, defer=False):
        """The weight-streaming kernel for at most 64 rows; k is split over workgroups when the
        output is too narrow to fill the GPU.  defer: the partial sums are returned as a SplitSum
        (or the finished tensor, where k is not split)."""
        tiles = (n + 15) // 16
        # many rows of x: the partial sums weigh more, and the waves do more work each
        target = self.skinny_target_waves if m <= 16 else self.skinny_target_waves // 2
        # few rows of x: staging them costs little, and four waves that share rows of the weight and
        # split k between them inside the workgroup leave fewer partial sums to add
        # (a gate/up product of up to 16 rows: two waves share the rows, which makes waves enough to
        # leave k unsplit, so that the gating happens in the product kernel and no partial sums are written)
        # (a long k, as in a down projection: two waves share the rows at every row count up to 16)
        kw = self.skinny_waves_per_tile or (2 if k >= 8192 and m <= 16 else 4 if m <= 4 else
                                            2 if swiglu and bias is None and m <= 16 else 1)
        splits = max(1, min((target + tiles * kw - 1) // (tiles * kw), k // 256))
        if swiglu and bias is None and 2 * tiles * kw >= target:
            splits = 1          # wide enough without a split of k: the gating happens in the product kernel
        if defer and splits == 1:
            defer = False
            out = torch.empty((m, n), dtype=x.dtype, device=x.device)
            os_ = n
        direct = splits == 1 and bias is None
        scratch = None if direct else torch.empty(splits * m * n, dtype=torch.float32, device=x.device)
        used = ctypes.c_int(0)
        library.call("gemm_skinny", "bf16", "nva_linear_skinny", _p(x), c_i64(xs), _p(weight), c_i64(ws),
                     None if defer else _p(bias), _p(out), c_i64(os_), c_i32(1 if out_float32 else 0),
                     c_i32(int(swiglu)), _p(scratch), c_i32(splits), c_i32(kw), c_i32(1 if defer else 0), c_i64(m), c_i64(n),
                     c_i64(k), ctypes.byref(used), self._stream())
        if defer:
            return SplitSum(self, scratch, used.value, m, n, bias)
        return out

    def _medium_shape(self, m: int, blocks: int, k: int):
        """(waves, row tiles, ranges of k) of the kernel for up to 256 rows, for a weight of `blocks`
        blocks of 16 rows.  A CU draws about its share of the memory's bandwidth and no more, so the
        product takes as long as its most loaded CU: of the workgroup sizes the kernel is built with
        (3 or 4 waves of 1 to 3 blocks each, fewer choices for many rows of x) the one is taken whose
        workgroups spread most evenly over the CUs; a weight of few blocks takes the largest
        workgroups and is split over k instead, into as many ranges as give at most one workgroup per
        CU (a second, partly filled round of workgroups costs more than CUs left idle)."""
        if self.medium_shape is not None:
            return self.medium_shape
        cus = self.medium_target_workgroups
        mb = ((m + 15) // 16 + 1) // 2 * 2
        if mb > 14:
            sizes = [(4, 1)]
        elif mb > 6:
            sizes = [(4, 2), (4, 1)]
        else:
            sizes = [(4, 2), (3, 3), (4, 3), (3, 2), (4, 1), (3, 1)]
        if self.medium_row_tiles == 1:
            sizes = [s for s in sizes if s[1] == 1] or sizes
        waves, rt = sizes[0]
        wgs = (blocks + waves * rt - 1) // (waves * rt)
        if 2 * wgs <= cus:
            return waves, rt, max(1, min(cus // wgs, k // 256))        # a weight of few blocks: split over k
        best = None
        for waves, rt in sizes:
            wgs = (blocks + waves * rt - 1) // (waves * rt)
            # rows (of the weight, and of x once per workgroup) that the most loaded CU streams
            cost = (((wgs + cus - 1) // cus) * (16 * waves * rt + m), -waves * rt)
            if best is None or cost < best[0]:
                best = (cost, waves, rt, 1)
        return best[1], best[2], best[3]

    def _linear_medium(self, x, xs, weight, ws, bias, out, os_, out_float32, swiglu, m, n, k, defer=False):
        """The weight-streaming kernel for up to 256 rows (see _linear_skinny for the arguments)."""
        blocks = (n // 2 + 7) // 8 if swiglu and bias is None and not defer else (n + 15) // 16
        waves, rt, splits = self._medium_shape(m, blocks, k)
        if defer and splits == 1:
            defer = False
            out = torch.empty((m, n), dtype=x.dtype, device=x.device)
            os_ = n
        direct = splits == 1 and bias is None
        scratch = None if direct else torch.empty(splits * m * n, dtype=torch.float32, device=x.device)
        used = ctypes.c_int(0)
        library.call("gemm_skinny", "bf16", "nva_linear_medium", _p(x), c_i64(xs), _p(weight), c_i64(ws),
                     None if defer else _p(bias), _p(out), c_i64(os_), c_i32(1 if out_float32 else 0),
                     c_i32(int(swiglu)), _p(scratch), c_i32(splits), c_i32(rt), c_i32(waves), c_i32(1 if defer else 0),
                     c_i64(m), c_i64(n), c_i64(k), ctypes.byref(used), self._stream())
        if defer:
            return SplitSum(self, scratch, used.value, m, n, bias)
        return out

    @staticmethod
    def _tile_takes(x, xs, weight, ws, m, n, k) -> bool:
        """The limits of nva_linear_tile: k in chunks of 64, 32-bit offsets into both operands."""
        return k % 64 == 0 and (m * xs + k) * 2 < 2 ** 32 and (n * ws + k) * 2 < 2 ** 32

    def _tile_plan(self, m: int, n: int, k: int, gated: bool, may_split: bool):
        """(shape, stages, ranges of k) of the LDS-tiled kernel: the tile of rows that holds all m (64,
        128 or 256; beyond that 256 and a grid dimension), 128 rows of the weight, as many stages as
        LDS holds, and, where the result may stay as partial sums, k cut into as many ranges as give
        about one workgroup per CU."""
        if self.tile_shape is not None:
            return tuple(self.tile_shape) + (0,) * (4 - len(self.tile_shape))
        shape, stages = (1, 3) if m <= 64 else (2, 3) if m <= 128 else (3, 4)     # (64 rows: two workgroups fit a CU)
        tiles = ((n // 2 if gated else n) + (63 if gated else 127)) // (64 if gated else 128)
        ranges = 1
        if may_split and not gated:
            ranges = max(1, min(self.teams // max(tiles, 1), k // 256))
        return shape, stages, ranges, self._tile_cols(m, n // 2 if gated else n, 64 if gated else 128, ranges)

    def _tile_cols(self, m: int, cols: int, tile_cols: int, ranges: int) -> int:
        """Columns of the result that a workgroup of the LDS-tiled kernel takes (0: its whole tile).  A CU
        draws its share of the memory's bandwidth and no more, so a weight is streamed fastest when every
        CU gets as many of its rows as every other: where whole tiles would make a second round that
        few CUs work in, or leave many CUs idle, the workgroups take as many columns each as shares
        the weight out evenly over the CUs in as many rounds (14B gate/up, 272 tiles on 256 CUs: 84
        instead of 105 µs at 64 rows, 153 instead of 164 at 256; 32B, 400 tiles: 111 instead of 116; 4B,
        152 tiles: 25 instead of 29).  Not where three quarters of the CUs have a tile anyway (8B
        gate/up, 192 tiles: the same time either way), not for a single round of more than 128 rows of x
        (every workgroup fetches all of x, and more workgroups fetch it more often: 72 instead of 65 µs
        there at 256 rows), and not for many rounds, which the hardware hands out evenly by itself (the
        head, 1187 tiles: 3 % slower)."""
        if self.tile_even_shares is False or ranges > 1:
            return 0
        tiles = (cols + tile_cols - 1) // tile_cols
        rounds = (tiles + self.cus - 1) // self.cus
        if tiles % self.cus == 0 or rounds > 2 or (rounds == 1 and (m > 128 or 10 * tiles > 7 * self.cus)):
            return 0
        share = ((cols + rounds * self.cus - 1) // (rounds * self.cus) + 7) // 8 * 8
        return share if share < tile_cols else 0

    def _linear_tile(self, x, xs, weight, ws, bias, out, os_, out_float32, swiglu, m, n, k, defer=False):
        """The LDS-tiled kernel for 17 rows and more (see _linear_skinny for the arguments)."""
        gated = bool(swiglu and bias is None and not defer)
        shape, stages, ranges, cols = self._tile_plan(m, n, k, gated, may_split=not gated and not out_float32)
        if swiglu and not gated:
            raise KernelError("linear_tile: the gated form takes no bias and is never deferred")
        if ranges == 1:
            if defer:
                defer = False
                out = torch.empty((m, n), dtype=x.dtype, device=x.device)
                os_ = n
            # (the gated form by its activation: swiglu is True or 1 for silu, 2 relu, 3 gelu)
            mode = (2 if int(swiglu) == 1 else 2 + int(swiglu)) if gated else 1 if out_float32 else 0
            library.call("gemm_tile", "bf16", "nva_linear_tile", _p(x), c_i64(xs), _p(weight), c_i64(ws), _p(bias), _p(out),
                         c_i64(os_), None, c_i32(mode), c_i64(m), c_i64(n), c_i64(k), c_i32(shape), c_i32(stages), c_i32(1),
                         c_i32(cols), None, self._stream())
            return out
        scratch = torch.empty(ranges * m * n, dtype=torch.float32, device=x.device)
        used = ctypes.c_int(0)
        library.call("gemm_tile", "bf16", "nva_linear_tile", _p(x), c_i64(xs), _p(weight), c_i64(ws), None, None, c_i64(0),
                     _p(scratch), c_i32(3), c_i64(m), c_i64(n), c_i64(k), c_i32(shape), c_i32(stages), c_i32(ranges),
                     c_i32(cols), ctypes.byref(used), self._stream())
        sums = SplitSum(self, scratch, used.value, m, n, bias)
        if defer:
            return sums
        library.call("gemm_skinny", "bf16", "nva_linear_skinny_finish", _p(scratch), c_i32(used.value), _p(bias), _p(out),
                     c_i64(os_), c_i32(1 if out_float32 else 0), c_i32(0), c_i64(m), c_i64(n), self._stream())
        return out

    def _linear_team(self, x, xs, weight, ws, bias, out, os_, mode, m, n, k):
        """The kernel for wide weights and at most 16 rows.  mode: 0 elements, 1 float, 2 gated."""
        library.call("gemm_team", "bf16", "nva_linear_team", _p(x), c_i64(xs), _p(weight), c_i64(ws), _p(bias), _p(out),
                     c_i64(os_), c_i32(mode), c_i64(m), c_i64(n), c_i64(k), c_i32(self.teams), self._stream())
        return out

    def linear_silu_mul(self, x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
        """silu(x @ Wg.T) * (x @ Wu.T) with weight = [Wg; Wu]."""
        return self.linear_act_mul(x, weight, "silu")

    def linear_act_mul(self, x: torch.Tensor, weight: torch.Tensor, act: str = "silu") -> torch.Tensor:
        """act(x @ Wg.T) * (x @ Wu.T) with weight = [Wg; Wu]; act: silu, relu or gelu_tanh.  The product
        kernels do the gating in their epilogues, whatever the activation."""
        if act not in self.ACTIVATIONS:
            raise KernelError(f"linear_act_mul: unknown activation {act!r}; known: {sorted(self.ACTIVATIONS)}")
        code = self.ACTIVATIONS[act]            # the kernels' gating flag is 1 + code, the team kernel's mode 2 + code
        x = _t(x)
        m, k, xs = _rows2d(x, "linear input")
        n, wk, ws = _rows2d(weight, "linear weight")
        if x.dtype == torch.bfloat16 and weight.dtype == x.dtype and wk == k and n % 2 == 0 and \
                self._own_kernel(m, n, k) == "team" and self._skinny_takes(x, xs, weight, ws, k):
            out = torch.empty((m, n // 2), dtype=x.dtype, device=x.device)
            return self._linear_team(x, xs, weight, ws, None, out, n // 2, 2 + code, m, n, k)
        if x.dtype == torch.bfloat16 and weight.dtype == x.dtype and wk == k and n % 2 == 0 and \
                self._skinny_takes(x, xs, weight, ws, k):
            own = self._own_kernel(m, n, k, gated=True)
            if own == "tile" and not self._tile_takes(x, xs, weight, ws, m, n, k):
                own = None
            if own in ("skinny", "medium", "tile"):
                out = torch.empty((m, n // 2), dtype=x.dtype, device=x.device)
                run = self._linear_skinny if own == "skinny" else self._linear_medium if own == "medium" else self._linear_tile
                run(x, xs, weight, ws, None, out, n // 2, False, 1 + code, m, n, k)
                return out
            if m > self.own_matmul_rows and (n, k, True) in self.product_choice:
                return self.act_mul(torch.nn.functional.linear(x, weight), act)      # measured: the library here
        return self.act_mul(self.linear(x, weight), act)

    # ------------------------------------------------------------------ position encoding
    def rotary_table(self, inv_freq: torch.Tensor, num_positions: int) -> torch.Tensor:
        """float32 [positions, 2 * len(inv_freq)]: cos(p * f) then sin(p * f)."""
        if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous():
            raise KernelError("rotary_table: inv_freq must be contiguous float32")
        half = inv_freq.shape[0]
        table = torch.empty((num_positions, 2 * half), dtype=torch.float32, device=inv_freq.device)
        library.call("rope", self.suffix, "nva_rotary_table", _p(inv_freq), c_i32(half), c_i64(num_positions), _p(table),
                     self._stream())
        return table

    def rotary_step_table(self, inv_freq: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """float32 [tokens, 2 * len(inv_freq)]: cos(p_t * f), then sin(p_t * f), for the step's tokens at their
        positions p_t (int32, read on the device)."""
        if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous():
            raise KernelError("rotary_step_table: inv_freq must be contiguous float32")
        tokens = positions.shape[0]
        _i32(positions, tokens, "positions")
        half = inv_freq.shape[0]
        table = torch.empty((tokens, 2 * half), dtype=torch.float32, device=inv_freq.device)
        library.call("rope", self.suffix, "nva_rotary_step_table", _p(inv_freq), c_i32(half), _p(positions), c_i64(tokens),
                     _p(table), self._stream())
        return table

    def qk_norm_rope_store(self, qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                           q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                           table: Optional[torch.Tensor], positions: Optional[torch.Tensor],
                           slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                           v_cache: Optional[torch.Tensor], max_position: Optional[int] = None) -> torch.Tensor:
        """Per-head norm of q and k, rotation by the table's rows, q and k written back in
        place, k and v written into their page slots.  Returns the q view [T, heads*head_dim].
        max_position: every entry of `positions` lies below it (the caller knows the step's
        largest position on the host); needed with a table, whose rows the kernel reads unchecked."""
        if table is not None:
            check_positions_fit(table, head_dim, max_position)
        if isinstance(qkv, SplitSum):
            return self._qk_of_partials(qkv, num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps, table,
                                        positions, slots, k_cache, v_cache)
        qkv = _t(qkv)
        tokens, width, stride = _rows2d(qkv, "qkv")
        if width != (num_heads + 2 * num_kv_heads) * head_dim:
            raise KernelError(f"qkv width {width} is not (heads + 2*kv_heads) * head_dim = "
                              f"{(num_heads + 2 * num_kv_heads) * head_dim}")
        wf = 0
        for w in (q_weight, k_weight):
            if w is not None:
                wf = self._norm_weight(w, head_dim, qkv)
        if num_kv_heads and (q_weight is None) != (k_weight is None):
            raise KernelError("qk norm: give both weights or none")
        if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
            raise KernelError("qk norm: the two weights differ in type")
        if table is not None:
            _i32(positions, tokens, "positions")
        page_size = 0
        if k_cache is not None:
            page_size = self._check_cache(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype)
            _i32(slots, tokens, "slots")
        library.call("rope", _suffix(qkv), "nva_qk_norm_rope_store", _p(qkv), c_i64(stride), c_i64(tokens),
                     c_i32(num_heads), c_i32(num_kv_heads), c_i32(head_dim), _p(q_weight), _p(k_weight), c_i32(wf),
                     c_f32(eps), _p(table), c_i32(0 if table is None else table.shape[1]), _p(positions), _p(slots),
                     _p(k_cache), _p(v_cache), c_i32(page_size), self._stream())
        return qkv[:, : num_heads * head_dim]

    def _qk_of_partials(self, qkv: "SplitSum", num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps, table,
                        positions, slots, k_cache, v_cache) -> torch.Tensor:
        tokens, width = qkv.shape
        if width != (num_heads + 2 * num_kv_heads) * head_dim:
            raise KernelError("qkv width is not (heads + 2*kv_heads) * head_dim")
        wf = 0
        for w in (q_weight, k_weight):
            if w is not None:
                wf = self._norm_weight(w, head_dim, qkv)
        if num_kv_heads and (q_weight is None) != (k_weight is None):
            raise KernelError("qk norm: give both weights or none")
        if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
            raise KernelError("qk norm: the two weights differ in type")
        if table is not None:
            _i32(positions, tokens, "positions")
        page_size = 0
        if k_cache is not None:
            page_size = self._check_cache(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype)
            _i32(slots, tokens, "slots")
        q = torch.empty((tokens, num_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
        library.call("rope", "bf16", "nva_qk_norm_rope_store_of_partials", _p(qkv.sums), c_i32(qkv.splits),
                     c_i64(tokens * width), _p(qkv.bias), _p(q), c_i64(num_heads * head_dim), c_i64(tokens),
                     c_i32(num_heads), c_i32(num_kv_heads), c_i32(head_dim), _p(q_weight), _p(k_weight), c_i32(wf),
                     c_f32(eps), _p(table), c_i32(0 if table is None else table.shape[1]), _p(positions), _p(slots),
                     _p(k_cache), _p(v_cache), c_i32(page_size), self._stream())
        return q

    def qk_rownorm_store(self, qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                         q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                         positions: Optional[torch.Tensor], temp_coef: float, temp_every: int,
                         slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                         v_cache: Optional[torch.Tensor], rot_table: Optional[torch.Tensor] = None,
                         norm_per_head: bool = False, rot_interleaved: bool = False, v_norm: bool = False,
                         v_first_in: Optional[torch.Tensor] = None, v_mix: Optional[torch.Tensor] = None,
                         v_first_out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """rot_interleaved: the rotation pairs the neighbours (2i, 2i + 1).  v_norm: every value head divided by its root
        mean square (eps, no weight).  v_first_out, float32 [tokens, kv_heads * v_head_dim]: receives the values after the
        norm.  v_first_in (the same shape) with v_mix (float32, one number on the device): v <- (1 - v_mix) v + v_mix
        v_first_in before the store.
        norm_per_head: the two norms run over every head by itself, with weights [head_dim] that the heads share.
        rot_table, float32 [tokens, rot]: after norm and temperature the first rot channels of every head
        of q and k are rotated in pairs (i, i + rot / 2) by the token's row (rot / 2 cosines, then sines).
        q and k normed over the whole projection (all heads at once, plain weights [heads * head_dim]
        and [kv_heads * head_dim]), q scaled by the temperature 1 + temp_coef * ln(floor((p + 1) /
        temp_every) + 1) of its position p, both written back in place, k and v written into their page
        slots.  The row is [q | k | v] with values of v_head_dim.  Returns the q view."""
        partial = isinstance(qkv, SplitSum) and self.fuse_split_sums
        if partial:
            (tokens, width), stride = qkv.shape, 0
        else:
            qkv = _t(qkv)
            tokens, width, stride = _rows2d(qkv, "qkv")
        want = (num_heads + num_kv_heads) * head_dim + num_kv_heads * v_head_dim
        if width != want:
            raise KernelError(f"qkv width {width} is not heads * head_dim + kv_heads * (head_dim + v_head_dim) = {want}")
        wf = 0
        for w, n in ((q_weight, num_heads * head_dim), (k_weight, num_kv_heads * head_dim)):
            if w is not None:
                wf = self._norm_weight(w, head_dim if norm_per_head else n, qkv)
        if num_kv_heads and (q_weight is None) != (k_weight is None):
            raise KernelError("qk norm: give both weights or none")
        if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
            raise KernelError("qk norm: the two weights differ in type")
        if temp_coef:
            if positions is None or int(temp_every) <= 0:
                raise KernelError("a query temperature needs the positions and a positive step")
            _i32(positions, tokens, "positions")
        rot = 0
        if rot_table is not None:
            rot = rot_table.shape[1] if rot_table.dim() == 2 else 0
            if rot_table.dtype != torch.float32 or rot_table.dim() != 2 or rot_table.shape[0] != tokens or \
                    not rot_table.is_contiguous() or rot <= 0 or rot % 2 or rot > head_dim:
                raise KernelError(f"qk_rownorm_store: the rotation table must be contiguous float32 [{tokens}, rot], rot "
                                  f"even and at most the head's {head_dim}")
        page_size = 0
        if k_cache is not None:
            page_size = self._check_cache(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype, v_head_dim)
            _i32(slots, tokens, "slots")
        vd = num_kv_heads * v_head_dim
        for name, vf in (("v_first_in", v_first_in), ("v_first_out", v_first_out)):
            if vf is not None and (vf.dtype != torch.float32 or tuple(vf.shape) != (tokens, vd) or not vf.is_contiguous()):
                raise KernelError(f"qk_rownorm_store: {name} must be contiguous float32 [{tokens}, {vd}]")
        if v_first_in is not None and (v_mix is None or v_mix.dtype != torch.float32 or v_mix.numel() != 1 or
                                       v_first_out is not None):
            raise KernelError("qk_rownorm_store: mixing values needs one float32 factor, and reads or writes the first values")
        if partial:
            # the projection's partial sums (and bias) are added up by the kernel; q gets a tensor of its own
            q = torch.empty((tokens, num_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
            source = [None, c_i64(0), _p(qkv.sums), c_i32(qkv.splits), c_i64(tokens * width), _p(qkv.bias), _p(q),
                      c_i64(num_heads * head_dim)]
        else:
            q = qkv[:, : num_heads * head_dim]
            source = [_p(qkv), c_i64(stride), None, c_i32(0), c_i64(0), None, _p(qkv), c_i64(stride)]
        library.call("qk_rownorm", "bf16" if partial else _suffix(qkv), "nva_qk_rownorm_store", *source, c_i64(tokens),
                     c_i32(num_heads), c_i32(num_kv_heads), c_i32(head_dim), c_i32(v_head_dim), _p(q_weight), _p(k_weight),
                     c_i32(wf), c_f32(eps), _p(positions), c_f32(float(temp_coef)), c_i32(int(temp_every) if temp_coef else 1),
                     _p(rot_table), c_i32(rot), _p(slots), _p(k_cache), _p(v_cache), c_i32(page_size),
                     c_i32(1 if norm_per_head and q_weight is not None else 0), c_i32(1 if rot_interleaved else 0),
                     c_i32(1 if v_norm else 0), _p(v_first_in), _p(v_mix) if v_first_in is not None else None,
                     _p(v_first_out), self._stream())
        return q

    def sigmoid_mul(self, x: torch.Tensor, gate: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x * sigmoid(gate), entry by entry, in float and rounded once; in place unless out is given."""
        x, gate = _t(x), _t(gate)
        rows, width, xs = _rows2d(x, "sigmoid_mul input")
        grows, gw, gs = _rows2d(gate, "sigmoid_mul gate")
        if (grows, gw) != (rows, width) or gate.dtype != x.dtype:
            raise KernelError("sigmoid_mul: the gate does not match the input")
        out = x if out is None else out
        orows, ow, os_ = _rows2d(out, "sigmoid_mul output")
        if (orows, ow) != (rows, width) or out.dtype != x.dtype:
            raise KernelError("sigmoid_mul: output does not match the input")
        library.call("activation", _suffix(x), "nva_sigmoid_mul", _p(x), c_i64(xs), _p(gate), c_i64(gs), _p(out), c_i64(os_),
                     c_i64(rows), c_i32(width), self._stream())
        return out

    @staticmethod
    def _check_cache(k_cache, v_cache, num_kv_heads, head_dim, dtype, v_head_dim=None) -> int:
        if k_cache.dim() != 4 or v_cache is None or v_cache.dim() != 5:
            raise KernelError("cache tensors must be K [pages, kv_heads, page, head_dim] and "
                              "V [pages, kv_heads, page / vt, v_head_dim, vt]")
        pages, h, page_size, d = k_cache.shape
        vd = head_dim if v_head_dim is None else v_head_dim
        if (h, d) != (num_kv_heads, head_dim) or tuple(v_cache.shape) != v_cache_shape(pages, h, vd, page_size):
            raise KernelError(f"cache shapes K {tuple(k_cache.shape)} V {tuple(v_cache.shape)} do not fit "
                              f"{num_kv_heads} kv heads of {head_dim}")
        if not (k_cache.is_contiguous() and v_cache.is_contiguous()) or k_cache.dtype != dtype or v_cache.dtype != dtype:
            raise KernelError("cache tensors must be contiguous and of the activations' type")
        return page_size

    # ------------------------------------------------------------------ attention
    def paged_attention(self, q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                        k_cache: torch.Tensor, v_cache: torch.Tensor, batch, group: int, scale: float,
                        window: Optional[int] = None, out: Optional[torch.Tensor] = None,
                        v_head_dim: Optional[int] = None, sinks: Optional[torch.Tensor] = None,
                        chunk: Optional[int] = None, softcap: Optional[float] = None, keep_first: int = 0,
                        sigmoid_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """sigmoid_bias, float32 [heads]: no softmax; a visible key weighs sigmoid(score + sigmoid_bias[head]), and the
        weights are not normalised over the keys.
        chunk: a query at position p reads the keys from floor(p / chunk) * chunk on only.
        softcap: a score s (after the scale) becomes softcap * tanh(s / softcap).  keep_first (with a window):
        every query also reads the first keep_first positions of its sequence, however far back.
        Causal attention of the step's tokens over the cache.  `batch` is the step's
        StepBatch; `group` selects its block tables.  q [T, heads*head_dim] (rows may be strided).
        v_head_dim: the size of a head's values where it is not head_dim (the output is then
        [T, heads*v_head_dim]).  sinks, float32 [heads]: one more term exp(sink_h) in the denominator
        of head h's softmax, a key without a value that every query sees once."""
        q = _t(q)
        tokens, width, qs = _rows2d(q, "attention q")
        if width != num_heads * head_dim:
            raise KernelError("attention: q width is not heads * head_dim")
        v_dim = head_dim if v_head_dim is None else int(v_head_dim)
        if sinks is not None and (sinks.dtype != torch.float32 or sinks.shape != (num_heads,) or not sinks.is_contiguous()):
            raise KernelError(f"attention: sinks must be contiguous float32 [{num_heads}]")
        page_size = self._check_cache(k_cache, v_cache, num_kv_heads, head_dim, q.dtype, v_dim)
        if num_heads % num_kv_heads:
            raise KernelError(f"attention: {num_heads} heads do not divide into {num_kv_heads} kv heads")
        tables = batch.groups[group].block_tables
        if tables.dtype != torch.int32 or tables.dim() != 2 or tables.shape[0] != batch.num_seqs or not tables.is_contiguous():
            raise KernelError("attention: block tables must be contiguous int32 [requests, pages]")
        _i32(batch.token_seq, tokens, "token_seq")
        _i32(batch.positions, tokens, "positions")
        need_pages = (batch.max_kv_len + page_size - 1) // page_size
        if tables.shape[1] < need_pages:
            raise KernelError(f"attention: block tables hold {tables.shape[1]} pages, {need_pages} are needed")
        if out is None:
            out = torch.empty((tokens, num_heads * v_dim), dtype=q.dtype, device=q.device)
        _, ow, os_ = _rows2d(out, "attention out")
        if ow != num_heads * v_dim or out.shape[0] != tokens or out.dtype != q.dtype:
            raise KernelError("attention: output does not match q")
        if any(n != 1 for n in batch.q_lens[:batch.num_decode]):
            raise KernelError("attention: the first num_decode requests of a batch must bring one token each")
        # tokens [0, num_decode) are single decoded tokens: the matrix-core decode kernel takes
        # them where its shape limits allow; everything else runs the general kernel
        start = 0
        # (the matrix-core kernels fold the scale into the exponent, which needs it positive)
        cap = float(softcap) if softcap else 0.0
        keep = int(keep_first) if window and keep_first else 0
        if cap < 0.0 or keep < 0:
            raise KernelError("attention: a negative softcap or number of kept positions")
        if sigmoid_bias is not None and (sigmoid_bias.dtype != torch.float32 or sigmoid_bias.shape != (num_heads,) or
                                         not sigmoid_bias.is_contiguous() or sinks is not None):
            raise KernelError(f"attention: sigmoid_bias must be contiguous float32 [{num_heads}] and goes without sinks")
        mfma = self.mfma_attention and q.dtype == torch.bfloat16 and 0.0 < scale < float("inf") and v_dim == head_dim
        if batch.num_decode > 0 and mfma and \
                self._decode_kernel_takes(num_heads // num_kv_heads, head_dim, page_size, q, qs, out, os_):
            start = batch.num_decode
            self._attention_decode(q, qs, out, os_, k_cache, v_cache, tables, batch, start, num_heads, num_kv_heads,
                                   head_dim, page_size, scale, window, sinks, chunk, keep, cap, sigmoid_bias)
        if batch.num_decode < tokens and mfma and \
                self._prefill_kernel_takes(head_dim, page_size, tables.shape[1], q, qs, out, os_):
            # portions of prompts: the matrix-core prefill kernel, one workgroup per 32 query rows
            tiles = self._prefill_tiles(batch, q.device)
            library.call("attn_prefill", "bf16", "nva_attn_prefill", _p(q), c_i64(qs), _p(out), c_i64(os_), _p(k_cache),
                         _p(v_cache), _p(tables), c_i32(tables.shape[1]), _p(batch.cu_seqlens_q), _p(batch.kv_lens),
                         _p(tiles), c_i64(tiles.shape[0]), c_i32(num_heads),
                         c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), c_f32(scale), c_i32(window or 0),
                         c_i32(chunk or 0), c_i32(keep), c_f32(cap), _p(sinks), _p(sigmoid_bias), _p(self.fault_flag),
                         self._stream())
            tokens = batch.num_decode            # what is left: the single tokens before the portions, if any
        if self.tiled_general_attention and start <= batch.num_decode < tokens and not window and sigmoid_bias is None and \
                max(head_dim, v_dim) <= GENERAL_TILED_MAX_HEAD_DIM:
            # portions of prompts in float arithmetic: the per-token kernel's arithmetic, operation for
            # operation, with the keys staged once for 32 query rows
            tiles = self._prefill_tiles(batch, q.device)
            library.call("attn_generic", _suffix(q), "nva_paged_attention_tiled", _p(q), c_i64(qs), _p(out), c_i64(os_),
                         _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]), _p(batch.cu_seqlens_q),
                         _p(batch.kv_lens), _p(tiles), c_i64(tiles.shape[0]), c_i32(num_heads), c_i32(num_kv_heads),
                         c_i32(head_dim), c_i32(v_dim), c_i32(page_size), c_f32(scale), c_i32(chunk or 0), c_f32(cap),
                         _p(sinks), _p(self.fault_flag), self._stream())
            tokens = batch.num_decode            # what is left: the single tokens before the portions
        if start < tokens:
            n = tokens - start
            # Few tokens with many keys each: a token's keys are shared out among several workgroups, a share of 128
            # keys or more, and a second kernel joins their results (a wave alone walks its keys one block after the
            # other).  The number of shares follows from the step's longest request and the number of tokens alone.
            reach = min(x for x in (batch.max_kv_len, (window + keep) if window else None, chunk) if x)
            # (Only where a cap or kept positions keep bfloat16 tokens from the matrix-core decode kernel: everywhere
            # else this kernel's sums keep the one order that the tiled form for portions shares, bit for bit.)
            shared = self.shared_general_attention and q.dtype == torch.bfloat16 and (cap > 0.0 or keep > 0) and \
                sigmoid_bias is None
            shares = max(1, min(16, reach // 128, 4096 // (n * num_heads))) if shared else 1
            part = torch.empty(n * num_heads * shares * (2 + v_dim), dtype=torch.float32, device=q.device) if shares > 1 else None
            library.call("attn_generic", _suffix(q), "nva_paged_attention_generic", _p(q[start:start + n]), c_i64(qs),
                         _p(out[start:]), c_i64(os_), _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]),
                         _p(batch.token_seq[start:]), _p(batch.positions[start:]), c_i64(n), c_i32(num_heads),
                         c_i32(num_kv_heads), c_i32(head_dim), c_i32(v_dim), c_i32(page_size), c_f32(scale),
                         c_i32(window or 0), c_i32(chunk or 0), c_i32(keep), c_f32(cap), _p(sinks), _p(sigmoid_bias), _p(part), c_i32(shares),
                         _p(self.fault_flag), self._stream())
        return out

    # ------------------------------------------------------------------ attention through a latent
    def latent_prepare(self, proj: torch.Tensor, heads: int, dim: int, rot: int, rank: int, weight: torch.Tensor, eps: float,
                       rot_table: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                       v_cache: Optional[torch.Tensor]) -> torch.Tensor:
        """proj [tokens, heads * (dim + rot) + rank + rot]: per head [dim plain | rot turned] query entries, then the
        token's raw latent and its raw turned key part.  The latent is normed (weight, eps), the turned parts are
        rotated in pairs of neighbours by rot_table (float32 [tokens, rot]: cosines, then sines); the cache's key row
        of the token becomes [latent | turned key part], its value row the latent.  Returns q2 [tokens, heads *
        (rank + rot)] with every head's turned part in its last rot entries; the first rank are left for the caller."""
        proj = _t(proj)
        tokens, width, stride = _rows2d(proj, "latent projection")
        if width != heads * (dim + rot) + rank + rot:
            raise KernelError(f"latent_prepare: a row of {width} is not heads * (dim + rot) + rank + rot")
        if rot_table.dtype != torch.float32 or tuple(rot_table.shape) != (tokens, rot) or not rot_table.is_contiguous():
            raise KernelError(f"latent_prepare: the rotation table must be contiguous float32 [{tokens}, {rot}]")
        wf = self._norm_weight(weight, rank, proj)
        page_size = 0
        if k_cache is not None:
            page_size = self._check_cache(k_cache, v_cache, 1, rank + rot, proj.dtype, rank)
            _i32(slots, tokens, "slots")
        q2 = torch.empty((tokens, heads * (rank + rot)), dtype=proj.dtype, device=proj.device)
        library.call("latent", _suffix(proj), "nva_latent_prepare", _p(proj), c_i64(stride), c_i64(tokens), c_i32(heads),
                     c_i32(dim), c_i32(rot), c_i32(rank), _p(weight), c_i32(wf), c_f32(eps), _p(rot_table), _p(q2),
                     c_i64(q2.shape[1]), _p(slots), _p(k_cache), _p(v_cache), c_i32(page_size), self._stream())
        return q2

    def latent_attention(self, q2: torch.Tensor, heads: int, rank: int, rot: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                         batch, group: int, scale: float, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Causal softmax attention of heads that share one key/value head whose key rows are [latent | rotated part]
        (rank + rot entries) and whose value rows are the latent: q2 [tokens, heads * (rank + rot)] -> [tokens, heads *
        rank].  bfloat16 with a latent of a multiple of 16 runs on the matrix cores (a token's heads are the columns of
        the products, so a key row is fetched once for all of them; a token's keys are shared out among workgroups
        where a step has few tokens); everything else runs the general attention kernel."""
        q2 = _t(q2)
        tokens, width, qs = _rows2d(q2, "latent attention q")
        page_size = self._check_cache(k_cache, v_cache, 1, rank + rot, q2.dtype, rank)
        if self.mfma_attention and q2.dtype == torch.bfloat16 and rank % 16 == 0 and 0 < rank <= 512 and rot % 8 == 0 and \
                0 < rot <= 128 and page_size % 32 == 0 and qs % 8 == 0 and 0.0 < scale < float("inf"):
            if width != heads * (rank + rot):
                raise KernelError("latent attention: q width is not heads * (rank + rot)")
            if sinks is not None and (sinks.dtype != torch.float32 or sinks.shape != (heads,) or not sinks.is_contiguous()):
                raise KernelError(f"latent attention: sinks must be contiguous float32 [{heads}]")
            tables = batch.groups[group].block_tables
            if tables.dtype != torch.int32 or tables.dim() != 2 or tables.shape[0] != batch.num_seqs or not tables.is_contiguous():
                raise KernelError("latent attention: block tables must be contiguous int32 [requests, pages]")
            if tables.shape[1] < (batch.max_kv_len + page_size - 1) // page_size:
                raise KernelError("latent attention: the block tables are too narrow for the step's longest request")
            _i32(batch.token_seq, tokens, "token_seq")
            _i32(batch.positions, tokens, "positions")
            out = torch.empty((tokens, heads * rank), dtype=q2.dtype, device=q2.device)
            if any(n != 1 for n in batch.q_lens[:batch.num_decode]):
                raise KernelError("latent attention: the first num_decode requests of a batch must bring one token each")
            single = batch.num_decode if tokens > batch.num_decode else tokens
            if single < tokens:
                # portions of prompts: four tokens in a row to a workgroup, the tiles of keys through LDS once for all four
                tiles = self._prefill_tiles(batch, q2.device)
                library.call("latent", "bf16", "nva_latent_attention_prefill", _p(q2), c_i64(qs), _p(out), c_i64(out.shape[1]),
                             _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]), _p(batch.cu_seqlens_q),
                             _p(batch.kv_lens), _p(tiles), c_i64(tiles.shape[0]), c_i32(heads), c_i32(rank), c_i32(rot),
                             c_i32(page_size), c_f32(scale), _p(sinks), _p(self.fault_flag), self._stream())
            if single > 0:
                # few tokens with many keys: a token's tiles of 32 keys are shared out, four tiles a share or more, until
                # about two waves a compute unit run; the number follows from the step's shape alone
                blocks = (heads + 15) // 16
                shares = max(1, min(64, ((batch.max_kv_len + 31) // 32) // 4, 512 // (single * blocks)))
                part = torch.empty(single * heads * shares * (2 + rank), dtype=torch.float32, device=q2.device) if shares > 1 else None
                library.call("latent", "bf16", "nva_latent_attention", _p(q2), c_i64(qs), _p(out), c_i64(out.shape[1]), _p(part),
                             c_i32(shares), _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]), _p(batch.token_seq),
                             _p(batch.positions), c_i64(single), c_i32(heads), c_i32(rank), c_i32(rot), c_i32(page_size),
                             c_f32(scale), _p(sinks), _p(self.fault_flag), self._stream())
            return out
        return self.paged_attention(q2, heads, 1, rank + rot, k_cache, v_cache, batch, group, scale, None, v_head_dim=rank,
                                    sinks=sinks)

    def heads_linear(self, x: torch.Tensor, x_head: int, w: torch.Tensor, heads: int, n_out: int, k_in: int,
                     transposed: bool, y: torch.Tensor, y_head: int, y_offset: int = 0) -> torch.Tensor:
        """A product per head: y[t, h * y_head + y_offset + n] = sum_k W[h][n][k] x[t, h * x_head + k], n < n_out, k < k_in.
        w is contiguous [heads * n_out, k_in], or with transposed [heads * k_in, n_out] (W[h][n][k] = w[h * k_in + k, n]).
        x and y are 2-d with rows of any stride.  Float sums over k in ascending order, rounded once (bfloat16 with
        matrices that are not transposed: on the matrix cores, in the order of their steps of 32)."""
        x = _t(x)
        tokens, xw, xs = _rows2d(x, "heads_linear input")
        yrows, yw, ys = _rows2d(y, "heads_linear output")
        if yrows != tokens or y.dtype != x.dtype or w.dtype != x.dtype or not w.is_contiguous() or \
                tuple(w.shape) != ((heads * k_in, n_out) if transposed else (heads * n_out, k_in)):
            raise KernelError("heads_linear: the output or the matrices do not fit the input")
        if (heads - 1) * x_head + k_in > xw or (heads - 1) * y_head + y_offset + n_out > yw or x_head < 0 or y_head < 0:
            raise KernelError("heads_linear: the heads do not fit the rows")
        w_n, w_k = (1, n_out) if transposed else (k_in, 1)
        yv = y[:, y_offset:] if y_offset else y
        if x.dtype == torch.bfloat16 and not transposed and k_in % 8 == 0 and xs % 8 == 0 and x_head % 8 == 0 and \
                x.data_ptr() % 16 == 0 and self.mfma_attention:
            library.call("latent", "bf16", "nva_heads_linear_mfma", _p(x), c_i64(xs), c_i64(x_head), _p(w), _p(yv), c_i64(ys),
                         c_i64(y_head), c_i64(tokens), c_i32(heads), c_i32(n_out), c_i32(k_in), self._stream())
            return y
        library.call("latent", _suffix(x), "nva_heads_linear", _p(x), c_i64(xs), c_i64(x_head), _p(w), c_i64(n_out * k_in),
                     c_i64(w_n), c_i64(w_k), _p(yv), c_i64(ys), c_i64(y_head), c_i64(tokens), c_i32(heads), c_i32(n_out),
                     c_i32(k_in), self._stream())
        return y

    # ------------------------------------------------------------------ delta rule
    def channel_delta(self, proj: torch.Tensor, decay_in: torch.Tensor, gate_in: torch.Tensor, heads: int, kv_heads: int,
                      dim: int, vdim: int, taps: int, conv_w: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
                      norm_w: torch.Tensor, eps: float, conv_state: torch.Tensor, s_state: torch.Tensor, batch,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The gated delta rule with a decay per key channel over the step's tokens: proj [T, 2 G D + H DV + H] =
        [q | k | v | b] with G = kv_heads heads of D = dim and H = heads heads of DV = vdim.  q, k, v pass a causal
        convolution of `taps` taps per channel (conv_w [C, taps]) and silu; q and k become unit vectors per head (q
        times D^-1/2); beta = sigmoid(b); a = exp(-exp(a_log) * softplus(decay_in + dt_bias)), decay_in float32
        [T, H D]; per head S <- diag(a) S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q; then o's RMS norm per head
        times norm_w [DV] times sigmoid(gate_in), gate_in [T, H DV].  s_state float32 [slots, H, D, DV] and conv_state
        float32 [slots, C, taps - 1] hold a request's state in the row batch.state_slots names, taken as zero where
        batch.seq_starts is 0.  Returns [T, H DV] of proj's type."""
        proj, gate_in = _t(proj), _t(gate_in)
        decay_in = _t(decay_in)
        tokens, width, stride = _rows2d(proj, "delta-rule projections")
        qk, vv, hd = kv_heads * dim, heads * vdim, heads * dim
        channels = 2 * qk + vv
        if width != channels + heads:
            raise KernelError(f"channel_delta: projections of width {width}, expected {channels + heads}")
        if decay_in.dtype != torch.float32 or tuple(decay_in.shape) != (tokens, hd) or not decay_in.is_contiguous():
            raise KernelError(f"channel_delta: the decay's input must be contiguous float32 [{tokens}, {hd}]")
        grows, gw, gs = _rows2d(gate_in, "delta-rule gate")
        if (grows, gw) != (tokens, vv) or gate_in.dtype != proj.dtype:
            raise KernelError("channel_delta: the gate's input does not match")
        if s_state.dtype != torch.float32 or tuple(s_state.shape[1:]) != (heads, dim, vdim) or not s_state.is_contiguous():
            raise KernelError(f"channel_delta: the state must be contiguous float32 [slots, {heads}, {dim}, {vdim}]")
        if conv_state.dtype != torch.float32 or tuple(conv_state.shape) != (s_state.shape[0], channels, taps - 1) or \
                not conv_state.is_contiguous():
            raise KernelError(f"channel_delta: the kept inputs must be contiguous float32 [slots, {channels}, {taps - 1}]")
        if tuple(conv_w.shape) != (channels, taps) or conv_w.dtype != proj.dtype or not conv_w.is_contiguous():
            raise KernelError("channel_delta: the convolution's weights do not fit")
        for v, n, what in ((dt_bias, hd, "dt_bias"), (a_log, heads, "a_log"), (norm_w, vdim, "norm_w")):
            if v.dtype != torch.float32 or tuple(v.shape) != (n,) or not v.is_contiguous():
                raise KernelError(f"channel_delta: {what} must be contiguous float32 [{n}]")
        seqs = batch.num_seqs
        _i32(batch.token_seq, tokens, "token_seq")
        _i32(batch.cu_seqlens_q, seqs + 1, "cu_seqlens_q")
        _i32(batch.seq_starts, seqs, "seq_starts")
        _i32(batch.state_slots, seqs, "state_slots")
        if sum(batch.q_lens) != tokens:
            raise KernelError("channel_delta: the batch does not describe the projections' rows")
        if out is None:
            out = torch.empty((tokens, vv), dtype=proj.dtype, device=proj.device)
        orows, ow, os_ = _rows2d(out, "delta-rule output")
        if (orows, ow) != (tokens, vv) or out.dtype != proj.dtype:
            raise KernelError("channel_delta: output does not match")
        dp = (dim + 3) // 4 * 4                         # rows of q, k and the decays are padded to whole float4s
        scratch = torch.empty(tokens * ((2 * kv_heads + heads) * dp + 2 * vv + heads), dtype=torch.float32, device=proj.device)
        library.call("delta", _suffix(proj), "nva_channel_delta", _p(proj), c_i64(stride), _p(decay_in), _p(gate_in), c_i64(gs),
                     _p(scratch), _p(out), c_i64(os_), _p(s_state), _p(conv_state if taps > 1 else None), _p(batch.token_seq),
                     _p(batch.cu_seqlens_q), _p(batch.seq_starts), _p(batch.state_slots), c_i64(seqs), c_i64(tokens),
                     c_i32(heads), c_i32(kv_heads), c_i32(dim), c_i32(vdim), c_i32(taps), _p(conv_w), _p(dt_bias), _p(a_log),
                     _p(norm_w), c_f32(eps), self._stream())
        return out

    # ------------------------------------------------------------------ state-space layer
    def state_space(self, proj: torch.Tensor, heads: int, vdim: int, n_state: int, groups: int, taps: int,
                    conv_w: torch.Tensor, conv_b: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
                    d_skip: torch.Tensor, norm_w: torch.Tensor, norm_groups: int, eps: float, conv_state: torch.Tensor,
                    ssm_state: torch.Tensor, batch, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A selective state-space layer over the step's tokens: proj [T, 2 H P + 2 G N + H] = [z | x B C | dt].
        x, B, C pass a causal convolution of `taps` taps per channel (conv_w [C, taps], conv_b [C]) and silu;
        dt <- softplus(dt + dt_bias); per head S <- exp(-exp(a_log) dt) S + dt B x^T, y = S^T C + d_skip x; then
        y * silu(z), an RMS norm in norm_groups parts, times norm_w.  ssm_state float32 [slots, H, N, P] and
        conv_state float32 [slots, C, taps - 1] hold a request's state in the row batch.state_slots names, taken
        as zero where batch.seq_starts is 0.  Returns [T, H P] of proj's type."""
        proj = _t(proj)
        tokens, width, stride = _rows2d(proj, "state-space projections")
        inner, gn = heads * vdim, groups * n_state
        channels = inner + 2 * gn
        if width != 2 * inner + 2 * gn + heads:
            raise KernelError(f"state_space: projections of width {width}, expected {2 * inner + 2 * gn + heads}")
        if ssm_state.dtype != torch.float32 or tuple(ssm_state.shape[1:]) != (heads, n_state, vdim) or not ssm_state.is_contiguous():
            raise KernelError(f"state_space: the state must be contiguous float32 [slots, {heads}, {n_state}, {vdim}]")
        if conv_state.dtype != torch.float32 or tuple(conv_state.shape) != (ssm_state.shape[0], channels, taps - 1) or \
                not conv_state.is_contiguous():
            raise KernelError(f"state_space: the kept inputs must be contiguous float32 [slots, {channels}, {taps - 1}]")
        if tuple(conv_w.shape) != (channels, taps) or tuple(conv_b.shape) != (channels,) or conv_w.dtype != proj.dtype or \
                conv_b.dtype != proj.dtype or not conv_w.is_contiguous() or not conv_b.is_contiguous():
            raise KernelError("state_space: the convolution's weights do not fit")
        for v, n, what in ((dt_bias, heads, "dt_bias"), (a_log, heads, "a_log"), (d_skip, heads, "d_skip"), (norm_w, inner, "norm_w")):
            if v.dtype != torch.float32 or tuple(v.shape) != (n,) or not v.is_contiguous():
                raise KernelError(f"state_space: {what} must be contiguous float32 [{n}]")
        seqs = batch.num_seqs
        _i32(batch.token_seq, tokens, "token_seq")
        _i32(batch.cu_seqlens_q, seqs + 1, "cu_seqlens_q")
        _i32(batch.seq_starts, seqs, "seq_starts")
        _i32(batch.state_slots, seqs, "state_slots")
        if sum(batch.q_lens) != tokens or any(n != 1 for n in batch.q_lens[:batch.num_decode]):
            raise KernelError("state_space: the batch does not describe the projections' rows (single tokens first)")
        if out is None:
            out = torch.empty((tokens, inner), dtype=proj.dtype, device=proj.device)
        orows, ow, os_ = _rows2d(out, "state-space output")
        if (orows, ow) != (tokens, inner) or out.dtype != proj.dtype:
            raise KernelError("state_space: output does not match")
        conv_out = torch.empty((tokens, channels), dtype=proj.dtype, device=proj.device)
        y_raw = torch.empty((tokens, inner), dtype=torch.float32, device=proj.device)
        # B and C once more as floats, in rows padded to what a thread of the recurrence holds, and (dt, decay) per head
        padded = getattr(library.load("ssd", self.suffix), f"nva_state_space_padded_rows_{self.suffix}")
        np_rows = int(padded(c_i32(n_state)))
        bc = torch.empty((tokens, groups, 2, np_rows), dtype=torch.float32, device=proj.device)
        if np_rows != n_state:
            bc.zero_()
        dtd = torch.empty((tokens, heads, 2), dtype=torch.float32, device=proj.device)
        # long portions are cut into blocks that run side by side (the same cut for every layer of the step)
        units = chains = block_states = cum = None
        n_units = n_chains = block_tokens = 0
        first = batch.num_decode
        if self.state_space_blocks_side_by_side and first < seqs:
            kept = getattr(batch, "step_cache", None)
            if kept is None:
                kept = batch.step_cache = {}
            plan = kept.get(("state_space_blocks", first, self.state_space_shape == 6))
            if plan is None:
                block_tokens, flat_units, flat_chains = (state_space_blocks if self.state_space_shape == 6 else retention_blocks)(
                    batch.q_lens, first)
                if flat_chains:
                    both = torch.tensor(flat_units + flat_chains, dtype=torch.int32).to(proj.device, non_blocking=True)
                    plan = (len(flat_units) // 4, len(flat_chains) // 4, both[: len(flat_units)], both[len(flat_units):],
                            block_tokens)
                else:
                    plan = (0, 0, None, None, 0)
                kept[("state_space_blocks", first, self.state_space_shape == 6)] = plan
            n_units, n_chains, units, chains, block_tokens = plan
            if n_chains:
                block_states = torch.empty((n_units, heads, n_state, vdim), dtype=torch.float32, device=proj.device)
                cum = torch.empty((tokens, heads), dtype=torch.float32, device=proj.device)
        library.call("ssd", _suffix(proj), "nva_state_space", _p(proj), c_i64(stride), _p(conv_out), _p(bc), _p(dtd), _p(y_raw),
                     _p(cum), _p(out),
                     c_i64(os_), _p(ssm_state), _p(conv_state), c_i64(ssm_state.shape[0]), _p(batch.token_seq),
                     _p(batch.cu_seqlens_q), _p(batch.seq_starts), _p(batch.state_slots), c_i64(seqs), c_i64(tokens),
                     c_i64(first), c_i32(heads), c_i32(vdim), c_i32(n_state), c_i32(groups), c_i32(taps), _p(conv_w),
                     _p(conv_b), _p(dt_bias), _p(a_log), _p(d_skip), _p(norm_w), c_i32(norm_groups), c_f32(eps), _p(units),
                     c_i64(n_units), _p(chains), c_i64(n_chains), c_i32(block_tokens), _p(block_states),
                     c_i32(self.state_space_shape),
                     self._stream())
        return out

    # ------------------------------------------------------------------ retention
    RETENTION_CHUNK = 32        # tokens of a chunk of nva_retention (the rows of its table of decay powers, less one)

    def retention(self, proj: torch.Tensor, heads: int, dim: int, v_dim: int, state: torch.Tensor,
                  decay_powers: torch.Tensor, inv_freq: Optional[torch.Tensor], k_scale: float, eps: float,
                  batch, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Retention of the step's tokens: proj [T, 2*heads*dim + 2*heads*v_dim] = [q | k | v | g];
        per head S <- decay S + k v^T, o = S^T q with q and k rotated by their position (inv_freq
        float32 [rot/2], None: no rotation) and k scaled by k_scale; then o / rms(o) * silu(g) per
        head.  state: float32 [slots, heads, dim, v_dim], a request's row given by batch.state_slots,
        started from zero where batch.seq_starts is 0.  decay_powers: float32 [heads, RETENTION_CHUNK + 1],
        decay_h^m.  Returns [T, heads*v_dim] of proj's type."""
        proj = _t(proj)
        tokens, width, stride = _rows2d(proj, "retention projections")
        if width != 2 * heads * (dim + v_dim):
            raise KernelError(f"retention: projections of width {width}, expected 2 * heads * (dim + v_dim) = "
                              f"{2 * heads * (dim + v_dim)}")
        if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, v_dim) or \
                not state.is_contiguous():
            raise KernelError(f"retention: the state must be contiguous float32 [slots, {heads}, {dim}, {v_dim}]")
        if decay_powers.dtype != torch.float32 or tuple(decay_powers.shape) != (heads, self.RETENTION_CHUNK + 1) or \
                not decay_powers.is_contiguous():
            raise KernelError(f"retention: decay powers must be contiguous float32 [{heads}, {self.RETENTION_CHUNK + 1}]")
        rot = 0
        if inv_freq is not None:
            if inv_freq.dtype != torch.float32 or inv_freq.dim() != 1 or not inv_freq.is_contiguous():
                raise KernelError("retention: inv_freq must be contiguous float32")
            rot = 2 * inv_freq.shape[0]
            if rot > dim:
                raise KernelError(f"retention: {rot} rotated channels of a head of {dim}")
        seqs = batch.num_seqs
        _i32(batch.cu_seqlens_q, seqs + 1, "cu_seqlens_q")
        _i32(batch.seq_starts, seqs, "seq_starts")
        _i32(batch.state_slots, seqs, "state_slots")
        if sum(batch.q_lens) != tokens or any(n != 1 for n in batch.q_lens[:batch.num_decode]):
            raise KernelError("retention: the batch does not describe the projections' rows (single tokens first)")
        if out is None:
            out = torch.empty((tokens, heads * v_dim), dtype=proj.dtype, device=proj.device)
        orows, ow, os_ = _rows2d(out, "retention output")
        if (orows, ow) != (tokens, heads * v_dim) or out.dtype != proj.dtype:
            raise KernelError("retention: output does not match")
        raw = torch.empty((tokens, heads * v_dim), dtype=torch.float32, device=proj.device)
        # value channels per workgroup: fewer where that is needed to give every CU a workgroup
        vslice = 32
        while vslice > 8 and seqs * heads * ((v_dim + vslice - 1) // vslice) < self.cus:
            vslice //= 2
        vslice = min(vslice, max(1, v_dim))
        positions = scratch = None
        if self.mfma_retention and rot and dim % 32 == 0 and dim <= 256 and v_dim % 32 == 0:
            _i32(batch.positions, tokens, "positions")
            positions = batch.positions
            scratch = torch.empty((tokens, rot), dtype=torch.float32, device=proj.device)
        # long portions are cut into blocks that run side by side (the same cut for every layer of the step)
        units = chains = block_states = None
        bt = n_units = n_chains = 0
        first = batch.num_decode if self.retention_decode_kernel else 0
        if self.mfma_retention and dim % 32 == 0 and dim <= 256 and v_dim % 32 == 0 and self.retention_blocks_side_by_side:
            kept = getattr(batch, "step_cache", None)
            if kept is None:
                kept = batch.step_cache = {}
            plan = kept.get(("retention_blocks", first))
            if plan is None:
                bt, flat_units, flat_chains = retention_blocks(batch.q_lens, first)
                if flat_chains:
                    both = torch.tensor(flat_units + flat_chains, dtype=torch.int32).to(proj.device, non_blocking=True)
                    plan = (bt, len(flat_units) // 4, len(flat_chains) // 4, both[: len(flat_units)], both[len(flat_units):])
                else:
                    plan = (0, 0, 0, None, None)
                kept[("retention_blocks", first)] = plan
            bt, n_units, n_chains, units, chains = plan
            if n_chains:
                block_states = torch.empty((n_units, heads, dim, v_dim), dtype=torch.float32, device=proj.device)
        library.call("retention", _suffix(proj), "nva_retention", _p(proj), c_i64(stride), _p(raw), _p(out), c_i64(os_),
                     _p(state), c_i64(state.shape[0]), _p(batch.cu_seqlens_q), _p(batch.seq_starts),
                     _p(batch.state_slots), c_i64(seqs), c_i64(tokens), _p(decay_powers), _p(inv_freq), c_i32(rot),
                     c_i32(heads), c_i32(dim), c_i32(v_dim), c_i32(vslice), c_f32(k_scale), c_f32(eps), _p(positions),
                     _p(scratch), c_i32(1 if self.mfma_retention else 0),
                     c_i64(first), _p(units), c_i64(n_units), _p(chains), c_i64(n_chains), c_i32(bt), _p(block_states),
                     self._stream())
        return out

    @staticmethod
    def batch_extras(q_lens, starts, num_decode) -> dict:
        """What these kernels want uploaded with a step's batch, from the step's shape alone (lengths
        and starts of the requests' portions, single tokens first): the order in which the prefill
        attention takes its tiles of 32 query rows.  Returned as {name: list of int}."""
        if num_decode == len(q_lens):
            return {}
        return {"prefill_tiles": prefill_tile_order(q_lens, starts, num_decode)}

    @staticmethod
    def _prefill_tiles(batch, device) -> torch.Tensor:
        """int32 [tiles, 2] = (request, tile of 32 query rows) of the step's portions of prompts, from the
        most keys to the fewest: uploaded with the batch where the batch's builder was given
        batch_extras, else made here, once per batch."""
        extras = getattr(batch, "extras", None)
        if extras is None:
            extras = batch.extras = {}
        tiles = extras.get("prefill_tiles")
        if tiles is None:
            flat = prefill_tile_order(batch.q_lens, batch.starts if getattr(batch, "starts", None) else
                                      [int(kv) - n for kv, n in zip(batch.kv_lens.tolist(), batch.q_lens)],
                                      batch.num_decode)
            tiles = torch.tensor(flat, dtype=torch.int32, device=device)
            extras["prefill_tiles"] = tiles
        if tiles.dtype != torch.int32 or tiles.numel() % 2 or not tiles.is_contiguous():
            raise KernelError("attention: prefill_tiles must be contiguous int32 [tiles, 2]")
        return tiles.view(-1, 2)

    @staticmethod
    def _decode_kernel_takes(group, head_dim, page_size, q, q_stride, out, out_stride) -> bool:
        """The limits of nva_attn_decode; what it does not take runs the general kernel."""
        return (group <= 16 and head_dim % 32 == 0 and 32 <= head_dim <= 256 and page_size % 8 == 0
                and q.data_ptr() % 16 == 0 and q_stride % 8 == 0 and out.data_ptr() % 16 == 0 and out_stride % 8 == 0)

    @classmethod
    def _prefill_kernel_takes(cls, head_dim, page_size, table_width, q, q_stride, out, out_stride) -> bool:
        """The limits of nva_attn_prefill (head sizes, page size, the block-table row it stages)."""
        return table_width <= PREFILL_MAX_TABLE and cls._decode_kernel_takes(1, head_dim, page_size, q, q_stride, out,
                                                                             out_stride)

    def _attention_decode(self, q, qs, out, os_, k_cache, v_cache, tables, batch, n, num_heads, num_kv_heads,
                          head_dim, page_size, scale, window, sinks=None, chunk=None, keep=0, cap=0.0, sigmoid_bias=None):
        # The work is shared out on the device from the tokens' positions, once per step and (kv
        # heads, window): the first layer that asks makes the plan, the others find it on the batch.
        # The library says how large the partial results may get for this many tokens of at most
        # max_kv_len keys, and how many persistent waves to launch.  At most 1024 tokens a launch.
        plans = getattr(batch, "step_cache", None)         # emptied by the model at the start of every pass
        if plans is None:
            plans = batch.step_cache = {}
        for t0 in range(0, n, 1024):
            t1 = min(n, t0 + 1024)
            key = ("decode_plan", t0, num_kv_heads, head_dim, page_size, window or 0, chunk or 0, keep)
            if key not in plans:
                bound, waves, ints = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int64(0)
                library.call("attn_decode", "bf16", "nva_attn_decode_plan_size", c_i32(batch.max_kv_len), c_i64(t1 - t0),
                             c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), c_i32(keep), ctypes.byref(bound),
                             ctypes.byref(waves), ctypes.byref(ints))
                plan = torch.empty(ints.value, dtype=torch.int32, device=q.device)
                library.call("attn_decode", "bf16", "nva_attn_decode_plan", _p(batch.positions[t0:t1]),
                             _p(batch.token_seq[t0:t1]), c_i64(t1 - t0),
                             c_i32(num_kv_heads), c_i32(page_size), c_i32(window or 0), c_i32(chunk or 0), c_i32(keep),
                             c_i32(bound.value), c_i32(waves.value), _p(plan), _p(self.fault_flag), self._stream())
                plans[key] = (plan, bound.value, waves.value)
            plan, bound, waves = plans[key]
            scratch = torch.empty(bound * num_heads * (head_dim + 2), dtype=torch.float32, device=q.device)
            library.call("attn_decode", "bf16", "nva_attn_decode", _p(q[t0:t1]), c_i64(qs), _p(out[t0:t1]), c_i64(os_),
                         _p(scratch), _p(plan), _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]),
                         c_i64(t1 - t0), c_i32(num_heads),
                         c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), c_f32(scale), c_f32(cap),
                         c_i32(bound), c_i32(waves), _p(sinks), _p(sigmoid_bias), _p(self.fault_flag), self._stream())

    # ------------------------------------------------------------------ sampling
    def sample(self, logits: torch.Tensor, temperatures: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
        """int32 [rows]: argmax where temperature is 0, else a draw from softmax(logits / T)
        with the row's counter-based noise key (int64 bit pattern of a 64-bit key)."""
        rows, vocab, stride = _rows2d(logits, "logits")
        if logits.dtype != torch.float32:
            raise KernelError("sample: logits must be float32")
        if temperatures.dtype != torch.float32 or temperatures.shape != (rows,) or not temperatures.is_contiguous():
            raise KernelError("sample: temperatures must be float32 [rows]")
        if keys.dtype != torch.int64 or keys.shape != (rows,) or not keys.is_contiguous():
            raise KernelError("sample: keys must be int64 [rows]")
        if rows > 65535:
            raise KernelError("sample: at most 65535 rows a call")
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        need = library.load("sample", None).nva_sample_scratch_bytes
        need.restype = ctypes.c_int64
        scratch = torch.empty((int(need(c_i64(rows), c_i32(vocab))) + 7) // 8, dtype=torch.float64, device=logits.device)
        library.call("sample", None, "nva_sample", _p(logits), c_i64(stride), c_i64(rows), c_i32(vocab),
                     _p(temperatures), _p(keys), _p(out), _p(scratch), self._stream())
        return out

    def advance_decode(self, batch, sampled: torch.Tensor, out_row: torch.Tensor, n_real: int, page_size: int) -> None:
        """Turns the metadata of a decode step whose tokens were sampled into that of the next
        decode step of the same requests, in place on the device; out_row receives the tokens."""
        n_total = batch.num_seqs
        for t, name in ((batch.input_ids, "input_ids"), (batch.positions, "positions"), (batch.kv_lens, "kv_lens"),
                        (batch.seq_starts, "seq_starts")):
            _i32(t, n_total, name)
        _i32(sampled, n_real, "sampled")
        _i32(out_row, n_real, "out_row")
        groups = batch.groups
        if len(groups) > self.max_burst_groups:
            raise KernelError(f"advance_decode: at most {self.max_burst_groups} cache groups")
        ptr = ctypes.c_void_p * max(len(groups), 1)
        widths = (ctypes.c_int * max(len(groups), 1))(*[g.block_tables.shape[1] for g in groups])
        for g in groups:
            _i32(g.slot_mapping, n_total, "slot_mapping")
            if g.block_tables.shape[0] != n_total or not g.block_tables.is_contiguous() or g.block_tables.dtype != torch.int32:
                raise KernelError("advance_decode: block tables must be contiguous int32 [requests, pages]")
        slots = ptr(*[g.slot_mapping.data_ptr() for g in groups])
        tables = ptr(*[g.block_tables.data_ptr() for g in groups])
        library.call("sample", None, "nva_advance_decode", _p(batch.input_ids), _p(batch.positions), _p(batch.kv_lens),
                     _p(batch.seq_starts), _p(sampled), _p(out_row), c_i32(n_real), c_i32(n_total),
                     c_i32(page_size), c_i32(len(groups)), slots, tables, widths, _p(self.fault_flag), self._stream())
