// Test infrastructure: decodes an image file with the stb_image.h the reference vendors
// (third_party/stb_image, the decoder examples/Res18/main.cpp:34 uses) and writes
// "width height channels\n" followed by the raw interleaved bytes to stdout.
#define STB_IMAGE_IMPLEMENTATION
#include "stb_image.h"

#include <cstdio>

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  int w = 0, h = 0, c = 0;
  unsigned char* d = stbi_load(argv[1], &w, &h, &c, 0);
  if (!d) return 1;
  printf("%d %d %d\n", w, h, c);
  fwrite(d, 1, (size_t)w * h * c, stdout);
  stbi_image_free(d);
  return 0;
}
