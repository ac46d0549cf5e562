"""Reader / writer of nncv's `model.bin` (the `-split-params` flat-array file).

Byte layout (little-endian, LP64), as written by nncv::rt::MemRefFlatArray::write
(src/libnncv/DataType.cpp:9-41) and utils::MemRefFlatBuffer::write
(src/nncv/compiler/Utils/BinaryParams.cpp:45-78):

    off 0   int64  magicNumber = 0x42
    off 8   uint64 memRefIndexStartOffset = 24
    off 16  uint64 numMemRefIndex = n
    off 24  n x MemRefIndexer (224 B): char name[128] | u64 dims | u64 shape[8] |
                                       u64 eleWidth | u64 aligned | u64 dataOffset
    then    tensor data, contiguous, row-major, indexer order, no padding

The reference pass skips fp16 constants (SplitParamsFlatArray.cpp:144-147); this writer extends
the format the natural way (eleWidth = 2), which the reference *reader* already accepts
(DataType.cpp:98-101).
"""
import struct

import numpy as np

MAGIC = 0x42
HEAD = struct.Struct("<qQQ")
INDEXER = struct.Struct("<128sQ8QQQQ")
assert HEAD.size == 24 and INDEXER.size == 224


def write(path, tensors, dtype=np.float32):
    """tensors: [(name, ndarray)]; every tensor is stored with element type `dtype`."""
    dtype = np.dtype(dtype)
    n = len(tensors)
    off = HEAD.size + n * INDEXER.size
    with open(path, "wb") as f:
        f.write(HEAD.pack(MAGIC, HEAD.size, n))
        arrs = []
        for name, a in tensors:
            a = np.ascontiguousarray(a, dtype=dtype)
            if a.ndim > 8:
                raise ValueError("rank > 8")
            shape = list(a.shape) + [0] * (8 - a.ndim)
            f.write(INDEXER.pack(name.encode()[:127], a.ndim, *shape, dtype.itemsize, 0, off))
            off += a.nbytes
            arrs.append(a)
        for a in arrs:
            f.write(a.tobytes())


def read(path, dtype=np.float32):
    """-> ([(name, shape, eleWidth)], flat blob of `dtype`).  Mirrors MemRefFlatArray::read
    (DataType.cpp:48-87): one blob of sum(numel*eleWidth) bytes read straight after the
    indexers; `dataOffset` is ignored.  Returns None on missing file or bad magic (the reference
    returns false); raises on a truncated file (the reference does not detect it)."""
    dtype = np.dtype(dtype)
    try:
        f = open(path, "rb")
    except OSError:
        return None
    with f:
        head = f.read(HEAD.size)
        if len(head) < HEAD.size:
            return None
        magic, start, n = HEAD.unpack(head)
        if magic != MAGIC:
            return None
        index, nbytes = [], 0
        for _ in range(n):
            name, dims, *rest = INDEXER.unpack(f.read(INDEXER.size))
            shape = tuple(rest[:dims])
            width = rest[8]
            index.append((name.split(b"\0", 1)[0].decode(), shape, width))
            nbytes += int(np.prod(shape, dtype=np.int64)) * width if dims else width
        blob = f.read(nbytes)
        if len(blob) != nbytes:
            raise IOError("model.bin truncated: %d of %d data bytes" % (len(blob), nbytes))
    return index, np.frombuffer(blob, dtype=dtype)


def write_resnet18(path, blob, dtype=np.float32):
    """Split a flat canonical-order parameter blob into named tensors and write it."""
    from . import resnet18_spec as spec
    blob = np.asarray(blob)
    assert blob.size == spec.NUM_ELEMENTS
    tensors, off = [], 0
    for name, shape in spec.tensor_table():
        k = spec.numel(shape)
        tensors.append((name, blob[off:off + k].reshape(shape)))
        off += k
    write(path, tensors, dtype)
