// Device-side helpers and the packed operand layout shared by every kernel of the
// W8A8 LoRA linear path (gfx950 only: wave64, MFMA, 160 KiB LDS).
//
// Packed int8 operand layout ("fragment order").  Both GEMM operands are stored as
// 1 KiB blocks of 32 rows (activation rows, or weight output columns) x 32 k.  Inside
// a block, lane l of a wavefront owns 16 consecutive bytes:
//     row-in-block = l % 32,   k-in-block = 16 * (l / 32) + byte
// which is exactly one v_mfma_i32_32x32x32_i8 A or B operand, so a wave fetches an
// operand with a single 16-byte-per-lane load of a contiguous 1 KiB chunk.  Blocks are
// ordered [row_block][k_block].  Weight columns are additionally permuted inside every
// group of 128: packed column 128g + 32j + c holds original column 128g + 4c + j, so a lane
// of the MFMA output owns four consecutive original columns (two (gate, up) pairs of a fused
// gate/up projection) in the four adjacent 32-column blocks of its wave.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w8a8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef unsigned short v8us __attribute__((ext_vector_type(8)));

constexpr int kBlk = 32;          // rows / columns / k per fragment block
constexpr int kBlockBytes = 1024; // bytes of one fragment block
constexpr int kTileM = 256;
constexpr int kTileN = 256;
constexpr int kTileK = 128;
constexpr int kMaxAdapters = 64;
constexpr int kMaxRank = 64;
constexpr int kMaxKSplit = 8;

__host__ __device__ inline uint32_t round_up(uint32_t v, uint32_t a) { return (v + a - 1) / a * a; }
__host__ __device__ inline uint32_t k_padded(uint32_t k) { return round_up(k, kTileK); }
__host__ __device__ inline uint32_t n_padded(uint32_t n) { return round_up(n, kTileN); }

// original weight column of packed column c
__host__ __device__ inline uint32_t packed_to_orig_col(uint32_t c) {
  return (c & ~127u) + 4u * (c & 31u) + ((c >> 5) & 3u);
}
// packed column of original column n (inverse of the above)
__host__ __device__ inline uint32_t orig_to_packed_col(uint32_t n) {
  return (n & ~127u) + 32u * (n & 3u) + ((n & 127u) >> 2);
}
// byte offset of element (row r, k) of a packed operand with kb k-blocks per row block
__host__ __device__ inline size_t packed_offset(uint32_t r, uint32_t k, uint32_t kb) {
  return ((size_t)(r >> 5) * kb + (k >> 5)) * kBlockBytes + ((r & 31u) + 32u * ((k & 31u) >> 4)) * 16u +
         (k & 15u);
}

__device__ inline float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// float pair -> packed bf16x2, round to nearest even (one v_cvt_pk_bf16_f32; NaN stays NaN)
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  const v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf));
}
// float -> bf16 bits, round to nearest even
__device__ inline uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.0f) & 0xffffu; }
__device__ inline float bf16_round_f32(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ inline double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt[3:0]|[15:14], expcnt[6:4], lgkmcnt[11:8])
template <int N>
__device__ inline void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}
__device__ inline void wait_vmcnt0() { wait_vmcnt<0>(); }

// Workgroup barrier for LDS hand-over that does not wait for outstanding global loads: the
// caller decides with wait_vmcnt<N>() how many direct-to-LDS loads may stay in flight.  The
// wave first drains its own LDS operations, so data it read is in registers and data it wrote
// is visible once every wave has passed.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// One wave copies 1 KiB: lane l moves 16 bytes global[src + 16 l] -> LDS[dst + 16 l].
__device__ inline void load_1k_to_lds(const unsigned char* src_lane, unsigned char* lds_dst_uniform) {
  __builtin_amdgcn_global_load_lds((gptr_t)src_lane, (lptr_t)lds_dst_uniform, 16, 0, 0);
}
// The same as an assembly statement the compiler keeps no books on (it treats the builtin as an access
// that may touch the LDS and then drains every counter at its next wait): lane l moves 16 bytes
// global[base + voff] -> LDS[lds_addr_uniform + 16 l]; inactive lanes move nothing.  The caller waits
// with s_waitcnt vmcnt and a barrier before the LDS is read.
// A gather of 64 dwords by one wave: lane l moves 4 bytes global[base + voff] (voff a multiple of 4, any
// place) -> LDS[lds_addr_uniform + 4 l].
__device__ inline void lds_gather_dword(const void* base_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(lds_addr_uniform) : "memory", "m0");
}
__device__ inline void lds_load_1k(const unsigned char* base_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base_uniform), "s"(lds_addr_uniform) : "memory", "m0");
}

}  // namespace w8a8
