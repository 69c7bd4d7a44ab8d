// Device sanity check, the counterpart of the reference's cuda_test target
// (src/cuda_test.cu: device properties + a vector add): lists the HIP devices
// the engine sees and pushes a 1 GiB copy through its plain copy kernel.
#include <cstdio>

#include "crl.h"

int main() {
  const int n = crl_device_count();
  if (n < 1) {
    std::printf("no HIP device: %s\n", crl_last_error());
    return 1;
  }
  std::printf("%d HIP device(s); engine version %s\n", n, crl_version());
  if (crl_probe_copy((size_t)1 << 30, 1) != CRL_OK) {
    std::printf("copy kernel failed: %s\n", crl_last_error());
    return 1;
  }
  std::printf("copy kernel ok\n");
  return 0;
}
