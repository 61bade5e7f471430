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

    def __init__(self, device="cuda:0", dtype: torch.dtype = torch.bfloat16, quiet: bool = False):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine runs on HIP kernels only and has no CPU path")
        if dtype not in _SUFFIX:
            raise KernelError(f"no kernels for element type {dtype}; bfloat16 and float32 are built")
        self.device = torch.device(device)
        self.dtype = dtype
        self.suffix = _SUFFIX[dtype]
        library.preload(self.suffix, quiet=quiet)       # compiles what this element type needs
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
        # False: the general kernel runs one wave per token for portions of prompts too (the same bits, slower)
        self.tiled_general_attention = True

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

    # ------------------------------------------------------------------ feed-forward
    def silu_mul(self, gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        gate_up = _t(gate_up)
        rows, width, xs = _rows2d(gate_up, "silu_mul input")
        if width % 2:
            raise KernelError("silu_mul: the input holds gate and up halves, its width must be even")
        inner = width // 2
        if out is None:
            out = torch.empty((rows, inner), dtype=gate_up.dtype, device=gate_up.device)
        orows, ow, os_ = _rows2d(out, "silu_mul output")
        if (orows, ow) != (rows, inner) or out.dtype != gate_up.dtype:
            raise KernelError("silu_mul: output does not match the input")
        library.call("activation", _suffix(gate_up), "nva_silu_mul", _p(gate_up), c_i64(xs), _p(out), c_i64(os_),
                     c_i64(rows), c_i32(inner), self._stream())
        return out

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
                     c_i32(1 if swiglu else 0), _p(scratch), c_i32(splits), c_i32(kw), c_i32(1 if defer else 0), c_i64(m), c_i64(n),
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
                     c_i32(1 if swiglu else 0), _p(scratch), c_i32(splits), c_i32(rt), c_i32(waves), c_i32(1 if defer else 0),
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
            mode = 2 if gated else 1 if out_float32 else 0
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
        x = _t(x)
        m, k, xs = _rows2d(x, "linear input")
        n, wk, ws = _rows2d(weight, "linear weight")
        if x.dtype == torch.bfloat16 and weight.dtype == x.dtype and wk == k and n % 2 == 0 and \
                self._own_kernel(m, n, k) == "team" and self._skinny_takes(x, xs, weight, ws, k):
            out = torch.empty((m, n // 2), dtype=x.dtype, device=x.device)
            return self._linear_team(x, xs, weight, ws, None, out, n // 2, 2, m, n, k)
        if x.dtype == torch.bfloat16 and weight.dtype == x.dtype and wk == k and n % 2 == 0 and \
                self._skinny_takes(x, xs, weight, ws, k):
            own = self._own_kernel(m, n, k, gated=True)
            if own == "tile" and not self._tile_takes(x, xs, weight, ws, m, n, k):
                own = None
            if own in ("skinny", "medium", "tile"):
                out = torch.empty((m, n // 2), dtype=x.dtype, device=x.device)
                run = self._linear_skinny if own == "skinny" else self._linear_medium if own == "medium" else self._linear_tile
                run(x, xs, weight, ws, None, out, n // 2, False, True, m, n, k)
                return out
            if m > self.own_matmul_rows and (n, k, True) in self.product_choice:
                return self.silu_mul(torch.nn.functional.linear(x, weight))      # measured: the library here
        return self.silu_mul(self.linear(x, weight))

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

    @staticmethod
    def _check_cache(k_cache, v_cache, num_kv_heads, head_dim, dtype) -> int:
        if k_cache.dim() != 4 or v_cache is None or v_cache.dim() != 5:
            raise KernelError("cache tensors must be K [pages, kv_heads, page, head_dim] and "
                              "V [pages, kv_heads, page / vt, head_dim, vt]")
        pages, h, page_size, d = k_cache.shape
        if (h, d) != (num_kv_heads, head_dim) or tuple(v_cache.shape) != v_cache_shape(pages, h, d, page_size):
            raise KernelError(f"cache shapes K {tuple(k_cache.shape)} V {tuple(v_cache.shape)} do not fit "
                              f"{num_kv_heads} kv heads of {head_dim}")
        if not (k_cache.is_contiguous() and v_cache.is_contiguous()) or k_cache.dtype != dtype or v_cache.dtype != dtype:
            raise KernelError("cache tensors must be contiguous and of the activations' type")
        return page_size

    # ------------------------------------------------------------------ attention
    def paged_attention(self, q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                        k_cache: torch.Tensor, v_cache: torch.Tensor, batch, group: int, scale: float,
                        window: Optional[int] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Causal attention of the step's tokens over the cache.  `batch` is the step's
        StepBatch; `group` selects its block tables.  q [T, heads*head_dim] (rows may be strided)."""
        q = _t(q)
        tokens, width, qs = _rows2d(q, "attention q")
        if width != num_heads * head_dim:
            raise KernelError("attention: q width is not heads * head_dim")
        page_size = self._check_cache(k_cache, v_cache, num_kv_heads, head_dim, q.dtype)
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
            out = torch.empty((tokens, width), dtype=q.dtype, device=q.device)
        _, ow, os_ = _rows2d(out, "attention out")
        if ow != width or out.shape[0] != tokens or out.dtype != q.dtype:
            raise KernelError("attention: output does not match q")
        if any(n != 1 for n in batch.q_lens[:batch.num_decode]):
            raise KernelError("attention: the first num_decode requests of a batch must bring one token each")
        # tokens [0, num_decode) are single decoded tokens: the matrix-core decode kernel takes
        # them where its shape limits allow; everything else runs the general kernel
        start = 0
        # (the matrix-core kernels fold the scale into the exponent, which needs it positive)
        mfma = self.mfma_attention and q.dtype == torch.bfloat16 and 0.0 < scale < float("inf")
        if batch.num_decode > 0 and mfma and \
                self._decode_kernel_takes(num_heads // num_kv_heads, head_dim, page_size, q, qs, out, os_):
            start = batch.num_decode
            self._attention_decode(q, qs, out, os_, k_cache, v_cache, tables, batch, start, num_heads, num_kv_heads,
                                   head_dim, page_size, scale, window)
        if start < tokens and mfma and start == batch.num_decode and \
                self._prefill_kernel_takes(head_dim, page_size, tables.shape[1], q, qs, out, os_):
            # portions of prompts: the matrix-core prefill kernel, one workgroup per 32 query rows
            tiles = self._prefill_tiles(batch, q.device)
            library.call("attn_prefill", "bf16", "nva_attn_prefill", _p(q), c_i64(qs), _p(out), c_i64(os_), _p(k_cache),
                         _p(v_cache), _p(tables), c_i32(tables.shape[1]), _p(batch.cu_seqlens_q), _p(batch.kv_lens),
                         _p(tiles), c_i64(tiles.shape[0]), c_i32(num_heads),
                         c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), c_f32(scale), c_i32(window or 0),
                         _p(self.fault_flag), self._stream())
            start = tokens
        if self.tiled_general_attention and start <= batch.num_decode < tokens and not window and \
                head_dim <= GENERAL_TILED_MAX_HEAD_DIM:
            # portions of prompts in float arithmetic: the per-token kernel's arithmetic, operation for
            # operation, with the keys staged once for 32 query rows
            tiles = self._prefill_tiles(batch, q.device)
            library.call("attn_generic", _suffix(q), "nva_paged_attention_tiled", _p(q), c_i64(qs), _p(out), c_i64(os_),
                         _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]), _p(batch.cu_seqlens_q),
                         _p(batch.kv_lens), _p(tiles), c_i64(tiles.shape[0]), c_i32(num_heads), c_i32(num_kv_heads),
                         c_i32(head_dim), c_i32(page_size), c_f32(scale), _p(self.fault_flag), self._stream())
            tokens = batch.num_decode            # what is left: the single tokens before the portions
        if start < tokens:
            n = tokens - start
            library.call("attn_generic", _suffix(q), "nva_paged_attention_generic", _p(q[start:start + n]), c_i64(qs),
                         _p(out[start:]), c_i64(os_), _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]),
                         _p(batch.token_seq[start:]), _p(batch.positions[start:]), c_i64(n), c_i32(num_heads),
                         c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), c_f32(scale), c_i32(window or 0),
                         _p(self.fault_flag), self._stream())
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
                          head_dim, page_size, scale, window):
        # The work is shared out on the device from the tokens' positions, once per step and (kv
        # heads, window): the first layer that asks makes the plan, the others find it on the batch.
        # The library says how large the partial results may get for this many tokens of at most
        # max_kv_len keys, and how many persistent waves to launch.  At most 1024 tokens a launch.
        plans = getattr(batch, "step_cache", None)         # emptied by the model at the start of every pass
        if plans is None:
            plans = batch.step_cache = {}
        for t0 in range(0, n, 1024):
            t1 = min(n, t0 + 1024)
            key = ("decode_plan", t0, num_kv_heads, head_dim, page_size, window or 0)
            if key not in plans:
                bound, waves, ints = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int64(0)
                library.call("attn_decode", "bf16", "nva_attn_decode_plan_size", c_i32(batch.max_kv_len), c_i64(t1 - t0),
                             c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), ctypes.byref(bound),
                             ctypes.byref(waves), ctypes.byref(ints))
                plan = torch.empty(ints.value, dtype=torch.int32, device=q.device)
                library.call("attn_decode", "bf16", "nva_attn_decode_plan", _p(batch.positions[t0:t1]),
                             _p(batch.token_seq[t0:t1]), c_i64(t1 - t0),
                             c_i32(num_kv_heads), c_i32(page_size), c_i32(window or 0), c_i32(bound.value),
                             c_i32(waves.value), _p(plan), _p(self.fault_flag), self._stream())
                plans[key] = (plan, bound.value, waves.value)
            plan, bound, waves = plans[key]
            scratch = torch.empty(bound * num_heads * (head_dim + 2), dtype=torch.float32, device=q.device)
            library.call("attn_decode", "bf16", "nva_attn_decode", _p(q[t0:t1]), c_i64(qs), _p(out[t0:t1]), c_i64(os_),
                         _p(scratch), _p(plan), _p(k_cache), _p(v_cache), _p(tables), c_i32(tables.shape[1]),
                         c_i64(t1 - t0), c_i32(num_heads),
                         c_i32(num_kv_heads), c_i32(head_dim), c_i32(page_size), c_f32(scale), c_i32(window or 0),
                         c_i32(bound), c_i32(waves), _p(self.fault_flag), self._stream())

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
