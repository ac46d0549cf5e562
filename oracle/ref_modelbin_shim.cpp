// C entry points over the reference's own nncv::rt::MemRefFlatArray
// (include/libnncv/DataType.hpp:164-196, src/libnncv/DataType.cpp:9-123), so that tests can ask
// the real reference reader/writer what a model.bin means.  Compiled together with the
// reference's DataType.cpp into oracle/_ref/ — test infrastructure only.
#include <cstring>
#include <new>
#include <string>

#include "libnncv/DataType.hpp"

using namespace nncv::rt;

extern "C" {

// Write `n` fp32 tensors with the reference writer.  shapes is n x 8, dims[i] gives the rank.
int ref_modelbin_write_f32(const char* path, int n, const char* const* names, const size_t* dims,
                           const size_t* shapes, float* const* data) {
  // The reference destructor deletes m_binaryData, which only read() ever sets
  // (DataType.cpp:121-123), so a write-only object is leaked rather than destroyed.
  auto* arr = new MemRefFlatArray(dataType::kFloat32);
  for (int i = 0; i < n; ++i) {
    MemRefIndexer ix;
    std::memset(&ix, 0, sizeof ix);
    std::strncpy(ix.name, names[i], sizeof(ix.name) - 1);
    ix.dims = dims[i];
    for (size_t d = 0; d < 8; ++d) ix.shape[d] = shapes[i * 8 + d];
    ix.eleWidth = 4;
    arr->addMemRefIndexer(ix, (void*)data[i]);
  }
  return arr->write(path) ? 0 : -1;
}

// Read with the reference reader; returns the total element count of the rank-1 descriptor it
// wraps (sizes[0]) or -1, and copies up to `cap` floats of the blob to `out`.
long long ref_modelbin_read_f32(const char* path, float* out, long long cap) {
  auto* arr = new MemRefFlatArray(dataType::kFloat32);  // leaked on purpose (see above)
  if (!arr->read(path)) return -1;
  auto* d = arr->getWrapedData<MemRefDescriptor<float, 1>>();
  long long n = d->sizes[0];
  if (d->offset != 0 || d->strides[0] != 1 || d->allocated != d->aligned) return -2;
  for (long long i = 0; i < n && i < cap; ++i) out[i] = d->aligned[i];
  return n;
}

size_t ref_sizeof_descriptor(int rank) {
  switch (rank) {
    case 1: return sizeof(MemRefDescriptor<float, 1>);
    case 2: return sizeof(MemRefDescriptor<float, 2>);
    case 4: return sizeof(MemRefDescriptor<float, 4>);
  }
  return 0;
}
size_t ref_sizeof_indexer() { return sizeof(MemRefIndexer); }
size_t ref_sizeof_head() { return sizeof(MemRefMagicHead); }
}
