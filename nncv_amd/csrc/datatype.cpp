// model.bin reader / writer and memref printer behind include/libnncv/DataType.hpp.
// File format: see nncv_amd/modelbin.py (same bytes as the reference's
// MemRefFlatArray::write/read, src/libnncv/DataType.cpp:9-87).
#include "libnncv/DataType.hpp"

#include <cstdio>
#include <cstring>
#include <iostream>

namespace nncv {
namespace rt {

namespace {
size_t elements_of(const MemRefIndexer& ix) {
  size_t n = 1;
  for (size_t d = 0; d < ix.dims && d < 8; ++d) n *= ix.shape[d];
  return n;
}
struct File {
  FILE* f;
  explicit File(const std::string& p, const char* mode) : f(fopen(p.c_str(), mode)) {}
  ~File() { if (f) fclose(f); }
};
}  // namespace

MemRefFlatArray::~MemRefFlatArray() {
  delete[] m_binaryData;
  switch (dataTypeWidth(m_dataType)) {  // the wrapper was allocated with the matching element type
    case 4: delete static_cast<MemRefDescriptor<nncvFloat32, 1>*>(m_wraped); break;
    case 2: delete static_cast<MemRefDescriptor<nncvFloat16, 1>*>(m_wraped); break;
    default: break;
  }
}

size_t MemRefFlatArray::numElements() const {
  size_t n = 0;
  for (const auto& ix : m_indexer) n += elements_of(ix);
  return n;
}

void MemRefFlatArray::addMemRefIndexer(const MemRefIndexer& indexer, void* data) {
  m_indexer.push_back(indexer);
  m_data.push_back(data);
}

bool MemRefFlatArray::write(const std::string& path) {
  if (m_data.size() != m_indexer.size()) return false;
  File out(path, "wb");
  if (!out.f) return false;
  m_head.magicNumber = 0x42;
  m_head.memRefIndexStartOffset = sizeof(MemRefMagicHead);
  m_head.numMemRefIndex = m_indexer.size();
  if (fwrite(&m_head, sizeof m_head, 1, out.f) != 1) return false;
  size_t cursor = sizeof(MemRefMagicHead) + m_indexer.size() * sizeof(MemRefIndexer);
  for (auto& ix : m_indexer) {
    ix.dataOffset = cursor;  // absolute file offset of this tensor's bytes
    if (fwrite(&ix, sizeof ix, 1, out.f) != 1) return false;
    cursor += elements_of(ix) * ix.eleWidth;
  }
  for (size_t i = 0; i < m_indexer.size(); ++i) {
    const size_t bytes = elements_of(m_indexer[i]) * m_indexer[i].eleWidth;
    if (bytes && fwrite(m_data[i], 1, bytes, out.f) != bytes) return false;
  }
  return fflush(out.f) == 0;
}

bool MemRefFlatArray::read(const std::string& path) {
  File in(path, "rb");
  if (!in.f) return false;
  if (fread(&m_head, sizeof m_head, 1, in.f) != 1) return false;
  if (m_head.magicNumber != 0x42) {
    printf("[ Erro ] The magic number of this %s bin file is broken\n", path.c_str());
    return false;
  }
  m_indexer.clear();
  m_data.clear();
  size_t bytes = 0;
  for (size_t i = 0; i < m_head.numMemRefIndex; ++i) {
    MemRefIndexer ix;
    if (fread(&ix, sizeof ix, 1, in.f) != 1 || ix.dims > 8) return false;
    bytes += elements_of(ix) * ix.eleWidth;
    m_indexer.push_back(ix);
  }
  delete[] m_binaryData;
  m_binaryData = new char[bytes ? bytes : 1];
  // the data section follows the index directly; dataOffset is informational
  if (bytes && fread(m_binaryData, 1, bytes, in.f) != bytes) {
    printf("[ Erro ] %s is shorter than its index says\n", path.c_str());
    return false;
  }
  size_t off = 0;
  for (const auto& ix : m_indexer) {
    m_data.push_back(m_binaryData + off);
    off += elements_of(ix) * ix.eleWidth;
  }
  wrap();
  return true;
}

void MemRefFlatArray::wrap() {
  const intptr_t total = (intptr_t)numElements();
  auto fill = [&](auto* d) {
    typedef decltype(d->aligned) P;
    d->allocated = d->aligned = reinterpret_cast<P>(m_binaryData);
    d->offset = 0;
    d->sizes[0] = total;
    d->strides[0] = 1;
    m_wraped = d;
  };
  switch (dataTypeWidth(m_dataType)) {
    case 4: fill(new MemRefDescriptor<nncvFloat32, 1>); break;
    case 2: fill(new MemRefDescriptor<nncvFloat16, 1>); break;
    default: m_wraped = nullptr; break;
  }
}

namespace {
void print_rec(std::ostream& os, const float* base, int64_t dim, int64_t rank, int64_t off, const intptr_t* sizes,
               const intptr_t* strides) {
  if (dim == rank) { os << base[off]; return; }
  os << "[";
  for (intptr_t i = 0; i < sizes[dim]; ++i) {
    if (i) os << (dim + 1 == rank ? ", " : ", \n");
    print_rec(os, base, dim + 1, rank, off + i * strides[dim], sizes, strides);
  }
  os << "]";
}
}  // namespace

extern "C" void printMemrefF32(int64_t rank, void* ptr) {
  auto* d = static_cast<MemRefDescriptor<float, 1>*>(ptr);
  const intptr_t* sizes = d->sizes;
  const intptr_t* strides = d->sizes + rank;
  std::cout << "Unranked Memref base@ = " << static_cast<const void*>(d->aligned) << " rank = " << rank
            << " offset = " << d->offset << " sizes = [";
  for (int64_t i = 0; i < rank; ++i) std::cout << (i ? ", " : "") << sizes[i];
  std::cout << "] strides = [";
  for (int64_t i = 0; i < rank; ++i) std::cout << (i ? ", " : "") << strides[i];
  std::cout << "] data = \n";
  print_rec(std::cout, d->aligned, 0, rank, d->offset, sizes, strides);
  std::cout << '\n' << std::flush;
}

}  // namespace rt
}  // namespace nncv
