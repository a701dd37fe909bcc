"""CPU oracle: what each tile / tensor op of the hot programs computes, one function per op name.

TEST INFRASTRUCTURE ONLY - see ``oracle/__init__.py``.

The reference gives every op a torch meaning in ``python/pypto/debug/torch_codegen.py:954-1128``
(the table) and ``:489-610`` (the helpers behind load / store / fillpad / assemble).  This module
restates those meanings for the 39 ops that the paged-attention, FFN, RMSNorm, projection and
paged-gather programs use - exactly the names the HIP target's op registry knows
(``pypto_amd.backend.registered_ops()``; the test holds the two sets equal) - so that

* a fused HIP kernel's claim "this op is realised here" can be checked against a stated meaning,
* the reference's kernels can be written out op by op (``tests/test_oracle_tile_ops.py`` does so for
  ``kernel_softmax_prepare``, its unaligned form, ``kernel_online_update``, the FFN's two kernels and
  RMSNorm) and compared with the stage-level and batched oracles.

A tile is a ``Tile``: a torch tensor plus the valid region ``tile.load`` recorded for it, which is what
``fillpad``, ``store`` and ``assemble`` look at (``_pypto_valid_shape`` in the reference's helpers).
Known-answer checks pin the parts a mistake could hide in: zero-padding of a load that reaches past
its source, the pad value of ``PadValue.min`` being the type's finite minimum, round-to-nearest-even
casts, ``keepdim`` reductions, and ``tile.matmul`` rounding its product to the operand type before
the cast to fp32 (``:1079``) - unlike the goldens, which accumulate in fp32.
"""

from __future__ import annotations

from typing import Callable, Sequence

import torch

from .attention import paged_gather as _paged_gather


class Tile:
    """A tensor with the valid region its load recorded (None = all of it)."""

    __slots__ = ("data", "valid")

    def __init__(self, data: torch.Tensor, valid: Sequence[int] | None = None) -> None:
        self.data = data
        self.valid = tuple(int(v) for v in valid) if valid is not None else None

    @property
    def shape(self) -> tuple[int, ...]:
        return tuple(self.data.shape)

    def valid_shape(self) -> tuple[int, ...]:
        return self.valid if self.valid is not None else self.shape


def _t(x):
    return x.data if isinstance(x, Tile) else x


def _like(x, data: torch.Tensor) -> Tile:
    """Element-wise results keep their first operand's valid region."""
    return Tile(data, x.valid if isinstance(x, Tile) else None)


# ---- data movement (torch_codegen.py:513-538, 577-610) ------------------------------------------
def load(tensor: torch.Tensor, offsets: Sequence[int], shapes: Sequence[int],
         valid_shape: Sequence[int] | None = None) -> Tile:
    """A ``shapes`` window of ``tensor`` at ``offsets``.  A window that reaches past the source is
    padded with zeros to the requested shape, and everything outside the valid region (given, or the
    part that exists) is zero as well (``_tile_load`` / ``_mask_valid_region``)."""
    window = tensor[tuple(slice(o, o + s) for o, s in zip(offsets, shapes))].clone()
    actual = tuple(window.shape)
    out = window.new_zeros(tuple(shapes))
    out[tuple(slice(0, s) for s in actual)] = window
    valid = tuple(min(v, a) for v, a in zip(valid_shape if valid_shape is not None else actual, actual))
    masked = out.new_zeros(tuple(shapes))
    region = tuple(slice(0, v) for v in valid)
    masked[region] = out[region]
    return Tile(masked, valid)


def store(tile, offsets: Sequence[int], output: torch.Tensor) -> torch.Tensor:
    """Writes the tile's valid region into ``output`` at ``offsets`` (``_tile_store``)."""
    t = tile if isinstance(tile, Tile) else Tile(tile)
    valid = t.valid_shape()
    output[tuple(slice(o, o + s) for o, s in zip(offsets, valid))] = t.data[tuple(slice(0, s) for s in valid)]
    return output


def fillpad(tile: Tile, pad_value: str = "zero") -> Tile:
    """Everything outside the valid region becomes 0, the type's finite minimum ("min") or its finite
    maximum ("max") - not an infinity (``_fillpad``, ``_pad_scalar`` :489-498)."""
    valid = tile.valid_shape()
    if valid == tile.shape:
        return Tile(tile.data.clone(), None)
    info = torch.finfo(tile.data.dtype) if tile.data.is_floating_point() else torch.iinfo(tile.data.dtype)
    fill = {"zero": 0, "min": info.min, "max": info.max}[pad_value]
    out = tile.data.new_full(tile.shape, fill)
    region = tuple(slice(0, v) for v in valid)
    out[region] = tile.data[region]
    return Tile(out, None)


def assemble(target: torch.Tensor, source, offsets: Sequence[int]) -> torch.Tensor:
    """The source's valid region written into ``target`` at ``offsets`` (``_assemble``)."""
    return store(source, offsets, target)


def move(tile, **_kw):
    """Between memory spaces: the same values (``_identity``)."""
    return tile


def create(shape: Sequence[int], dtype: torch.dtype = torch.float32) -> torch.Tensor:
    return torch.zeros(tuple(shape), dtype=dtype)


def full(shape: Sequence[int], value: float, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    return torch.full(tuple(shape), value, dtype=dtype)


def reshape(tile, shape: Sequence[int]):
    return _like(tile, _t(tile).reshape(tuple(shape))) if isinstance(tile, Tile) and tile.valid is None else \
        Tile(_t(tile).reshape(tuple(shape)))


def transpose_view(tile):
    """The trailing two dimensions swapped, no copy (``.mT``)."""
    return Tile(_t(tile).mT)


def slice_(tile, shape: Sequence[int], offsets: Sequence[int]):
    return Tile(_t(tile)[tuple(slice(o, o + s) for o, s in zip(offsets, shape))])


def read(container, index):
    """One element (``tensor.read`` / ``tile.read``): ``container[index]``."""
    return _t(container).reshape(-1)[index] if isinstance(index, int) else _t(container)[index]


def dim(tensor, axis: int) -> int:
    return _t(tensor).shape[axis]


# ---- arithmetic -------------------------------------------------------------------------------------
def _binary(fn: Callable) -> Callable:
    return lambda a, b: _like(a, fn(_t(a), _t(b)))


def _unary(fn: Callable) -> Callable:
    return lambda a, *_tmp: _like(a, fn(_t(a)))


add = _binary(torch.add)
sub = _binary(torch.sub)
mul = _binary(torch.mul)
maximum = _binary(torch.maximum)
adds = _binary(lambda a, s: a + s)   # scalar forms: the same arithmetic, broadcast
muls = _binary(lambda a, s: a * s)
neg = _unary(torch.neg)
exp = _unary(torch.exp)
sqrt = _unary(torch.sqrt)
rsqrt = _unary(torch.rsqrt)          # the tile form may carry a scratch tile, ignored (:1004)
recip = _unary(torch.reciprocal)
relu = _unary(torch.relu)           # :1071
# broadcasting forms: a [rows, cols] tile with a [rows, 1] column or a [1, cols] row
row_expand_sub = _binary(torch.sub)
row_expand_mul = _binary(torch.mul)
row_expand_div = _binary(torch.div)
col_expand_mul = _binary(torch.mul)


def cast(tile, target_type: torch.dtype):
    """``.to(dtype)``: round to nearest, ties to even (``_handle_cast``)."""
    return _like(tile, _t(tile).to(target_type))


def row_max(tile, *_tmp):
    """Per-row maximum, kept as a ``[rows, 1]`` column (``amax(dim=-1, keepdim=True)``)."""
    return Tile(_t(tile).amax(dim=-1, keepdim=True))


def row_sum(tile, *_tmp):
    return Tile(_t(tile).sum(dim=-1, keepdim=True))


def matmul(a, b):
    """``torch.matmul(a, b).float()``: the product is formed in the operands' type and only then cast
    (:1079).  With 16-bit operands this rounds every output to 16 bits, which the goldens do not."""
    return Tile(torch.matmul(_t(a), _t(b)).float())


def matmul_acc(acc, a, b):
    return Tile(_t(acc) + torch.matmul(_t(a), _t(b)).float())


def paged_gather(src, indices, block_table, block_size: int, col_offset: int = 0, size: int | None = None):
    """``out[i, :] = src[block_table[idx // bs] * bs + idx % bs, col_off : col_off + size]``
    (src/ir/op/tensor_ops/paged_gather.cpp:74-199)."""
    return _paged_gather(src, indices, block_table, block_size, src.shape[1] - col_offset if size is None else size,
                         col_offset)


def get_block_idx() -> int:
    """The block a kernel instance runs as under SPMD dispatch: 0 on the CPU (``:1068``), where one instance
    does all the work."""
    return 0


def get_block_num() -> int:
    """The number of SPMD instances.  The table gives this op no meaning; with the index fixed at 0 the
    only count under which ``for b in range(idx, batch, num)`` (09_paged_attention_spmd.py:129) still
    visits every sequence is 1."""
    return 1


# op name -> meaning.  The keys are the op registry's names.
TILE_OPS: dict[str, Callable] = {
    "tensor.create": create, "tensor.dim": dim, "tensor.paged_gather": paged_gather, "tensor.read": read,
    "tensor.slice": slice_,
    "tile.add": add, "tile.adds": adds, "tile.assemble": assemble, "tile.cast": cast,
    "tile.col_expand_mul": col_expand_mul, "tile.create": create, "tile.exp": exp, "tile.fillpad": fillpad,
    "tile.full": full, "tile.get_block_idx": get_block_idx, "tile.get_block_num": get_block_num, "tile.load": load, "tile.matmul": matmul, "tile.matmul_acc": matmul_acc,
    "tile.maximum": maximum, "tile.move": move, "tile.mul": mul, "tile.muls": muls, "tile.neg": neg,
    "tile.read": read, "tile.recip": recip, "tile.relu": relu, "tile.reshape": reshape, "tile.row_expand_div": row_expand_div,
    "tile.row_expand_mul": row_expand_mul, "tile.row_expand_sub": row_expand_sub, "tile.row_max": row_max,
    "tile.row_sum": row_sum, "tile.rsqrt": rsqrt, "tile.slice": slice_, "tile.sqrt": sqrt, "tile.store": store,
    "tile.sub": sub, "tile.transpose_view": transpose_view,
}
