// Runtime types of the nncv C ABI, source-compatible with the reference header of the same path
// (include/libnncv/DataType.hpp): a program written against nncv — e.g. examples/Res18/main.cpp —
// compiles against this file unchanged.  Only what that ABI needs is here:
//   MemRefDescriptor<T,N>   MLIR's strided memref struct              (reference :129-136)
//   MemRefIndexer / MemRefMagicHead   on-disk records of model.bin    (reference :144-162)
//   MemRefFlatArray          model.bin reader/writer + rank-1 wrapper  (reference :164-196)
//   DynamicMemRefType / wrapToIndexableTensor / At / printMemrefF32   result access helpers
// Written from the format, not from the reference's code: same layout, same member names, own
// implementation (bounds-checked reads, owned storage, no leaks).
#ifndef NNCV_LIB_NNCV_RT_DATA_TYPE_HPP_
#define NNCV_LIB_NNCV_RT_DATA_TYPE_HPP_

// the reference header pulls these in and callers (examples/Res18/main.cpp) rely on it
#include <array>
#include <cassert>
#include <cmath>
#include <complex>
#include <cstddef>
#include <cstdint>
#include <iomanip>
#include <initializer_list>
#include <iostream>
#include <memory>
#include <string>
#include <vector>

namespace nncv {
namespace rt {

enum class dataType : size_t { kFloat32 = 0x1, kFloat16, kInt32, kInt16, kUnknow };

typedef int16_t nncvInt16;
typedef int32_t nncvInt32;
typedef uint32_t nncvFloat32;
typedef uint16_t nncvFloat16;

template <typename T, size_t N>
struct MemRefDescriptor {
  T* allocated;
  T* aligned;
  intptr_t offset;
  intptr_t sizes[N];
  intptr_t strides[N];
};

template <typename T>
struct UnrankedMemRefType {
  int64_t rank;
  void* descriptor;
};

struct MemRefIndexer {  // 224 bytes on disk
  char name[128];
  size_t dims;
  size_t shape[8];
  size_t eleWidth;
  size_t aligned;
  size_t dataOffset;
};

struct MemRefMagicHead {  // 24 bytes on disk
  int64_t magicNumber = 0x42;
  size_t memRefIndexStartOffset;
  size_t numMemRefIndex;
};

static_assert(sizeof(MemRefIndexer) == 224 && sizeof(MemRefMagicHead) == 24, "model.bin record sizes");
static_assert(sizeof(MemRefDescriptor<float, 1>) == 40 && sizeof(MemRefDescriptor<float, 2>) == 56 &&
                  sizeof(MemRefDescriptor<float, 4>) == 88,
              "memref descriptor sizes");

inline size_t dataTypeWidth(dataType dt) {
  switch (dt) {
    case dataType::kFloat32: case dataType::kInt32: return 4;
    case dataType::kFloat16: case dataType::kInt16: return 2;
    default: return 0;
  }
}

class MemRefFlatArray {
 public:
  MemRefFlatArray() = delete;
  explicit MemRefFlatArray(const dataType& dt) : m_dataType(dt) {}
  ~MemRefFlatArray();
  MemRefFlatArray(const MemRefFlatArray&) = delete;
  MemRefFlatArray& operator=(const MemRefFlatArray&) = delete;

  // false on missing file, bad magic, or (unlike the reference) a file shorter than its index says
  bool read(const std::string& path);
  bool write(const std::string& path);
  void addMemRefIndexer(const MemRefIndexer& indexer, void* data);

  template <typename T>
  inline T* getWrapedData() { return (T*)m_wraped; }
  // MemRefDescriptor<elem,1>* over the whole blob: sizes[0] = total element count
  inline void* get() { return m_wraped; }

  // extensions
  const std::vector<MemRefIndexer>& indexers() const { return m_indexer; }
  size_t numElements() const;

 private:
  void wrap();
  MemRefMagicHead m_head{};
  std::vector<MemRefIndexer> m_indexer;
  std::vector<void*> m_data;
  dataType m_dataType;
  void* m_wraped = nullptr;
  char* m_binaryData = nullptr;
};

// Rank-erased view used to index a result: dmt[At{i, j}]
template <typename T>
class DynamicMemRefType {
 public:
  explicit DynamicMemRefType(const UnrankedMemRefType<T>& m) : rank(m.rank) {
    auto* d = static_cast<MemRefDescriptor<T, 1>*>(m.descriptor);
    basePtr = d->allocated;
    data = d->aligned;
    offset = d->offset;
    sizes = d->sizes;            // sizes[rank] is followed directly by strides[rank]
    strides = d->sizes + rank;
  }
  T& operator[](std::initializer_list<int> at) {
    int64_t lin = offset, k = 0;
    for (int i : at) lin += (int64_t)i * strides[k++];
    return data[lin];
  }
  int64_t rank;
  T* basePtr;
  T* data;
  int64_t offset;
  const intptr_t* sizes;
  const intptr_t* strides;
};

template <typename T>
DynamicMemRefType<T> wrapToIndexableTensor(int64_t rank, void* ptr) {
  UnrankedMemRefType<T> u = {rank, ptr};
  return DynamicMemRefType<T>(u);
}

typedef std::initializer_list<int> At;

extern "C" void printMemrefF32(int64_t rank, void* ptr);

}  // namespace rt
}  // namespace nncv

#endif  // NNCV_LIB_NNCV_RT_DATA_TYPE_HPP_
