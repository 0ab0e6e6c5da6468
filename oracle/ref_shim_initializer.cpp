// C entry point around the reference's own table initialiser so that tests can call it through ctypes.
// Compiled TOGETHER WITH the reference's csrc/utils/initializer.cu (read in place from the reference
// tree, never copied) against the thrust headers this image ships.  Test infrastructure only.
#include "utils/initializer.h" // the reference's header, found through -I<reference>/csrc

extern "C" void ref_initialize_host(float *data, unsigned long len, int type, float a, float b, unsigned int seed) {
  // type: 0 Zero, 1 Normal, 2 Uniform, 3 TruncatedNormal (order of hetuCTR::InitType, initializer.h:8-14)
  hetuCTR::Initializer init(static_cast<hetuCTR::InitType>(type), a, b);
  hetuCTR::initialize(data, len, init, /*host=*/true, seed);
}
