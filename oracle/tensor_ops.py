"""CPU oracle for ``raf.op.l2norm``, ``raf.op.fuse_tensor`` and ``raf.op.defuse_tensor`` --
TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests, the smoke check and the benchmark's CPU
baseline leg may import this module.

What is restated, and from where (paths relative to the reference tree):

* ``l2norm``: sqrt(sum(x*x)) over all elements, output a 0-d tensor of x's dtype
  (python/raf/_tvm_op/reduce.py:535-542; src/op/declare/reduce.cc:118-124; the cuBLAS backend
  calls nrm2, src/op/dialect/cublas/l2_norm.cc:57-71).  Evaluated in float64 and rounded once.
* ``fuse_tensor``: the tensors' bytes back to back in list order, result 1-d with the total element
  count and the first tensor's dtype (src/op/declare/memory.cc:43-63;
  src/op/dialect/cuda/memory.cc:55-68).
* ``defuse_tensor``: the inverse; ``sizes`` are element counts, ``shapes`` the concatenated
  dimensions and ``shape_indices`` the end position of each tensor's dimensions in ``shapes``
  (memory.cc:65-93; src/op/dialect/cuda/memory.cc:120-134).

Parity status: pinned (tests/test_oracle_tensor_ops.py) -- l2norm by exact rational sums of
squares on small inputs, Pythagorean closed forms, ``math.fsum`` and homogeneity; fuse/defuse by
element-by-element loops, round trips and the declared output shapes.
"""
from __future__ import annotations

from typing import List, Sequence

import numpy as np

from oracle.halfs import bf16_bits_to_f32, f32_to_bf16_bits


def l2norm_f64(x: np.ndarray) -> float:
    """sqrt(sum x_i^2) in float64; ``uint16`` input is taken as bfloat16 bit patterns."""
    x = np.asarray(x)
    if x.dtype == np.uint16:
        x = bf16_bits_to_f32(x)
    x64 = x.astype(np.float64).ravel()
    return float(np.sqrt(np.dot(x64, x64)))


def l2norm(x: np.ndarray) -> np.ndarray:
    """The op's result: a 0-d array of x's dtype (bfloat16: a 0-d uint16 bit pattern)."""
    x = np.asarray(x)
    r = l2norm_f64(x)
    if x.dtype == np.uint16:
        return f32_to_bf16_bits(np.array(r, dtype=np.float32)).reshape(())
    with np.errstate(over="ignore"):
        return np.array(r, dtype=np.float64).astype(x.dtype).reshape(())


def fuse_tensor(data: Sequence[np.ndarray]) -> np.ndarray:
    """Flat 1-d array holding every tensor's elements in list order."""
    assert len(data) > 0, "fuse_tensor of an empty list has no output (memory.cc:54-55)"
    dtype = data[0].dtype
    assert all(a.dtype == dtype for a in data), "one dtype for the whole list (memory.cc:58-60)"
    return np.concatenate([np.ascontiguousarray(a).ravel() for a in data])


def defuse_tensor(data: np.ndarray, sizes: Sequence[int], shapes: Sequence[int],
                  shape_indices: Sequence[int]) -> List[np.ndarray]:
    data = np.ascontiguousarray(data).ravel()
    assert sum(sizes) == data.size, f"Input tensor size should be {sum(sizes)}, got {data.size}."
    assert len(sizes) == len(shape_indices)
    out, start, dim0 = [], 0, 0
    for n, dim1 in zip(sizes, shape_indices):
        shape = tuple(int(d) for d in shapes[dim0:dim1])
        assert int(np.prod(shape, dtype=np.int64)) == n
        out.append(data[start:start + n].reshape(shape).copy())
        start += n
        dim0 = dim1
    return out


def defuse_args(data: Sequence[np.ndarray]):
    """(sizes, shapes, shape_indices) describing a tensor list the way the reference's callers
    build them for defuse_tensor."""
    sizes = [int(a.size) for a in data]
    shapes, idx = [], []
    for a in data:
        shapes.extend(int(d) for d in a.shape)
        idx.append(len(shapes))
    return sizes, shapes, idx
