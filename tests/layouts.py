"""Operand layouts (dims, strides, offset, storage size) used by the parity tests: the views the
reference's tensor layer produces — contiguous, sliced (offset), broadcast (stride 0),
transposed / permuted."""
import numpy as np


def contiguous(dims, off=0):
    s, acc = [], 1
    for d in reversed(dims):
        s.append(acc)
        acc *= d
    return dict(dims=list(dims), strides=list(reversed(s)), off=off, size=acc + off + (1 if off else 0))


def broadcast(dims, from_dims, off=0):
    """View of a contiguous tensor of shape from_dims (same rank, 1 where broadcast) as dims."""
    base = contiguous(from_dims)
    strides = [0 if f == 1 and d != 1 else st for d, f, st in zip(dims, from_dims, base["strides"])]
    return dict(dims=list(dims), strides=strides, off=off, size=int(np.prod(from_dims)) + off)


def permuted(dims, perm, off=0):
    """Logical shape dims obtained by permuting a contiguous tensor: logical dim i is storage dim perm[i]."""
    storage_dims = [0] * len(dims)
    for i, p in enumerate(perm):
        storage_dims[p] = dims[i]
    base = contiguous(storage_dims)
    strides = [base["strides"][p] for p in perm]
    return dict(dims=list(dims), strides=strides, off=off, size=int(np.prod(dims)) + off)


def gather(storage, lay):
    """Materialise the logical tensor a layout describes (numpy reference for index math)."""
    idx = np.zeros(lay["dims"], dtype=np.int64) + lay["off"]
    for ax, (d, s) in enumerate(zip(lay["dims"], lay["strides"])):
        shape = [1] * len(lay["dims"])
        shape[ax] = d
        idx = idx + (np.arange(d, dtype=np.int64) * s).reshape(shape)
    return storage[idx]
