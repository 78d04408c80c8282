// Skinny-M (decode) path: split-K streaming kernel.  Placeholder until the kernel lands.
#pragma once
#include "../../include/mi355_w8a8.h"
#include "w8a8_device.h"

namespace w8a8 {
constexpr int kSkinnyMaxRows = 32;
inline uint64_t skinny_workspace_bytes(uint32_t, uint32_t) { return 0; }
inline bool skinny_supported() { return false; }
inline int launch_skinny(const mi355_w8a8_problem*, unsigned char*, float*, uint16_t*, unsigned char*, uint32_t,
                         uint32_t, hipStream_t) {
  return MI355_W8A8_ERR_UNSUPPORTED;
}
}  // namespace w8a8
