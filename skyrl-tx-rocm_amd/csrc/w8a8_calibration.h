// Calibration kernels: what this part sustains on the two resources the path is priced against.
//   cal_mfma_kernel<SHAPE>: int8 MFMAs on operands that stay in registers (no LDS, no memory traffic
//     inside the timed loop), one wave per SIMD, 256 accumulator registers per lane.  SHAPE 0 is the
//     32 x 32 x 32 instruction (4 x 4 accumulator blocks), SHAPE 1 the 16 x 16 x 64 one (8 x 8 blocks).
//     The operands come from a buffer the caller fills: zeros, random bits or realistic codes.  The rate
//     depends on them, because the part runs into its power limit and lowers its clock with the number
//     of bits that toggle.
//   cal_read_kernel: a read-only stream over a buffer (16 bytes per lane and load, eight loads in flight).
//   cal_copy_kernel: a plain copy, for scaling hardware traffic counters.
// Each workgroup 17 also reports shader cycles and 100 MHz ticks of its timed loop, from which the
// caller gets the shader clock the run sustained.
#pragma once
#include "w8a8_device.h"

namespace w8a8 {

constexpr uint32_t kCalOperandBytes = 256u * 4u * 16u * 1024u;  // per workgroup and wave: 16 fragments of 1 KiB

template <int SHAPE>
__global__ __launch_bounds__(256, 1)
void cal_mfma_kernel(const unsigned char* __restrict__ operands, uint32_t iters, uint64_t* clocks, int32_t* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const v4i* frag = reinterpret_cast<const v4i*>(operands) + ((size_t)blockIdx.x * 4u + wave) * 16u * 64u + lane;
  int s = 0;
  long long c0, w0;
  if constexpr (SHAPE == 1) {
    v4i a[8], b[8], acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = frag[i * 64]; b[i] = frag[(8 + i) * 64]; }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = v4i{0, 0, 0, 0};
    c0 = clock64(); w0 = wall_clock64();
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) s += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  } else {
    v4i a[4], b[4];
    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { a[i] = frag[i * 64]; b[i] = frag[(8 + i) * 64]; }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    c0 = clock64(); w0 = wall_clock64();
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  }
  __builtin_amdgcn_s_waitcnt(0);
  const long long c1 = clock64(), w1 = wall_clock64();
  if (s == 0x7fffffff) sink[0] = s;  // keeps the accumulators alive; not taken on any real operand set
  if (blockIdx.x == 17 && threadIdx.x == 0) { clocks[0] = (uint64_t)(c1 - c0); clocks[1] = (uint64_t)(w1 - w0); }
}

constexpr uint32_t kCalGrid = 256;  // workgroups of four waves: one wave per SIMD of the 256 CUs

__global__ __launch_bounds__(256)
void cal_read_kernel(const v4i* __restrict__ src, uint64_t n16, uint32_t* sink) {
  // workgroup b reads the 32 KiB pieces b, b + gridDim.x, ...: 8 loads of 16 bytes per lane each
  v4i x = {0, 0, 0, 0};
  const uint64_t pieces = n16 / 2048u;
  for (uint64_t p = blockIdx.x; p < pieces; p += gridDim.x) {
    const v4i* q = src + p * 2048u + threadIdx.x;
    v4i v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = __builtin_nontemporal_load(q + i * 256);
#pragma unroll
    for (int i = 0; i < 8; ++i) x ^= v[i];
  }
  const int r = x[0] ^ x[1] ^ x[2] ^ x[3];
  if (r == 0x5a5a5a5a) sink[0] = (uint32_t)r;  // keeps the loads alive
}

// plain copy of n16 16-byte words: the kernel of known traffic that scales the FETCH_SIZE / WRITE_SIZE counters
__global__ __launch_bounds__(256)
void cal_copy_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, uint64_t n16) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256u) dst[i] = src[i];
}

}  // namespace w8a8
