// ResNet-18 driver with the flow of nncv's examples/Res18/main.cpp (read model.bin, fill a
// [B,3,H,W] input, normalise with the ImageNet mean/std, call _mlir_ciface_forward, time it,
// arg-max), minus the JPEG decoding: the image comes from a raw little-endian float32 file of
// B*3*H*W values in [0,1] (CHW), or is a synthetic gradient when no file is given.
//
//   clang++ -O2 -std=c++17 examples/res18_main.cpp -Iinclude -Lnncv_amd/lib -lnncv_hip \
//           -Wl,-rpath,$PWD/nncv_amd/lib -o res18
//   ./res18 model.bin [image.f32] [B H W]
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <vector>

#include "libnncv/DataType.hpp"

using namespace nncv::rt;

extern "C" void _mlir_ciface_forward(MemRefDescriptor<float, 2>* dst, MemRefDescriptor<float, 4>* src, void* params);

int main(int argc, char** argv) {
  const char* model = argc > 1 ? argv[1] : "model.bin";
  const char* image = argc > 2 ? argv[2] : nullptr;
  const int B = argc > 3 ? atoi(argv[3]) : 1, H = argc > 4 ? atoi(argv[4]) : 256, W = argc > 5 ? atoi(argv[5]) : 256;

  MemRefFlatArray params(dataType::kFloat32);
  if (!params.read(model)) {
    fprintf(stderr, "cannot read %s\n", model);
    return -1;
  }
  std::vector<float> x((size_t)B * 3 * H * W);
  if (image) {
    FILE* f = fopen(image, "rb");
    if (!f || fread(x.data(), sizeof(float), x.size(), f) != x.size()) {
      fprintf(stderr, "cannot read %zu floats from %s\n", x.size(), image);
      return -1;
    }
    fclose(f);
  } else {
    for (size_t i = 0; i < x.size(); ++i) x[i] = (float)((i * 2654435761u) % 1000) / 999.0f;
  }
  const float mean[3] = {0.485f, 0.456f, 0.406f}, stdv[3] = {0.229f, 0.224f, 0.225f};
  for (int b = 0; b < B; ++b)
    for (int c = 0; c < 3; ++c)
      for (int i = 0; i < H * W; ++i) {
        float& v = x[((size_t)b * 3 + c) * H * W + i];
        v = (v - mean[c]) / stdv[c];
      }

  MemRefDescriptor<float, 2> dst = {nullptr, nullptr, 0, {B, 1000}, {1000, 1}};
  MemRefDescriptor<float, 4> src = {x.data(), x.data(), 0, {B, 3, H, W}, {3 * H * W, H * W, W, 1}};

  for (int rep = 0; rep < 2; ++rep) {  // the first call uploads and prepares the weights
    auto t0 = std::chrono::steady_clock::now();
    _mlir_ciface_forward(&dst, &src, params.get());
    auto t1 = std::chrono::steady_clock::now();
    std::cout << (rep ? "Time: " : "Time (first call, with weight upload): ")
              << std::chrono::duration<double, std::milli>(t1 - t0).count() << "ms" << std::endl;
    if (rep == 0) free(dst.allocated);
  }
  auto out = wrapToIndexableTensor<float>(2, &dst);
  for (int b = 0; b < B; ++b) {
    int idx = 0;
    float best = out[At{b, 0}];
    for (int i = 1; i < 1000; ++i)
      if (out[At{b, i}] > best) {
        best = out[At{b, i}];
        idx = i;
      }
    std::cout << idx << std::endl;
  }
  free(dst.allocated);
  return 0;
}
