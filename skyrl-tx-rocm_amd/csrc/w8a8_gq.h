// Group-scaled quantized linear: W4 or W8 weights with one scale per (K group, output), A4 or A8
// activations with one scale per (row, K group) (skyrl/tx/kernels/quantized_lora.py:199-254, the
// general form whose group = K, 8-bit case the tiled and streaming kernels cover).
//
//   out[m, n] = sum_g ((f32(sum_{k in g} xq[m, k] wq[k, n]) * sx[m, g]) * sw[g, n])     groups in order
//               + s[idx[m]] * ((x @ A[idx[m]]) @ B[idx[m]])[m, n]                       float32, one cast
//
// Integer sums are exact; the float32 products and the sum over the groups are evaluated in the
// reference's order by one wave per output block, so the float32 base is reproduced bit for bit.
// int4 codes stay packed in HBM; they enter the int8 matrix core as 16 * code (the nibble moved to
// the high half of a byte), and the exact factor 1/16 is taken out after the scales.
//
//   gq_pack_weight_kernel  reference layout -> matrix-core fragments, 4-bit codes stay 4-bit
//   gq_quant_kernel        per (row, group): amax, scale, codes (row-major int8, rows padded to 32)
//   gq_lora_z_kernel       z = x @ A[idx] in float32
//   gq_gemm_kernel         one wave per 32 x 32 output block over all groups, epilogue, store
#pragma once
#include "w8a8_device.h"

namespace w8a8 {

// Packed weight: blocks of 32 columns x 32 k, ordered [column block][k block].  8-bit: 1 KiB, lane l
// holds column l % 32, k = 16 (l / 32) + 0..15 as 16 bytes.  4-bit: 512 bytes, lane l holds the same 16
// codes in 8 bytes: byte j of the first dword = code j (low nibble) and code 4 + j (high nibble), byte j
// of the second dword = code 8 + j and code 12 + j.
__host__ __device__ inline uint64_t gq_packed_bytes(uint32_t k_pad, uint32_t n, uint32_t bits) {
  return (uint64_t)((n + 31u) / 32u) * (k_pad / 32u) * (bits == 4u ? 512u : 1024u);
}

struct GqPackArgs {
  const unsigned char* codes;  // bits 8: int8 [k_pad, n]; bits 4: uint8 [k_pad / 2, n], low nibble = even k
  unsigned char* packed;
  uint32_t k_pad, n, bits;
  uint64_t n_items;            // column blocks * k blocks * 64 lanes
};

__device__ inline int gq_code_at(const GqPackArgs& a, uint32_t k, uint32_t col) {
  if (col >= a.n) return 0;
  if (a.bits == 8u) return (int)(int8_t)a.codes[(size_t)k * a.n + col];
  const uint32_t byte = a.codes[(size_t)(k >> 1) * a.n + col];
  return (int)((k & 1u) ? (byte >> 4) : (byte & 15u));  // the raw nibble: two's complement, kept as is
}

__global__ __launch_bounds__(256) void gq_pack_weight_kernel(GqPackArgs a) {
  const uint64_t item = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (item >= a.n_items) return;
  const uint32_t lane = (uint32_t)(item & 63u);
  const uint64_t blk = item >> 6;
  const uint32_t kbs = a.k_pad / 32u;
  const uint32_t nb = (uint32_t)(blk / kbs), kb = (uint32_t)(blk % kbs);
  const uint32_t col = nb * 32u + (lane & 31u), k0 = kb * 32u + 16u * (lane >> 5);
  if (a.bits == 8u) {
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) w[j >> 2] |= ((uint32_t)gq_code_at(a, k0 + j, col) & 0xffu) << (8u * (j & 3u));
    *reinterpret_cast<uint4*>(a.packed + blk * 1024u + lane * 16u) = make_uint4(w[0], w[1], w[2], w[3]);
  } else {
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
      w[0] |= ((uint32_t)gq_code_at(a, k0 + j, col) | ((uint32_t)gq_code_at(a, k0 + 4u + j, col) << 4)) << (8u * j);
      w[1] |= ((uint32_t)gq_code_at(a, k0 + 8u + j, col) | ((uint32_t)gq_code_at(a, k0 + 12u + j, col) << 4)) << (8u * j);
    }
    *reinterpret_cast<uint2*>(a.packed + blk * 512u + lane * 8u) = make_uint2(w[0], w[1]);
  }
}

// ---------------------------------------------------------------------------------------
struct GqQuantArgs {
  const uint16_t* x;   // bf16 [M, K]
  int8_t* codes;       // int8 [M_pad, K_pad]; rows >= M and columns >= K hold zeros
  float* scales;       // f32 [M_pad, G]
  uint32_t M, M_pad, K, K_pad, group, G;
  float qmax;          // 127 or 7
};

// scale = amax > 0 ? amax / qmax : 1, code = clip(rint(x / scale), -qmax, qmax), IEEE float32
// division, round half to even (quantized_lora.py:199-212).  One wave per row, group after group.
__global__ __launch_bounds__(256) void gq_quant_kernel(GqQuantArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= a.M_pad) return;
  const bool live = row < a.M;
  const uint16_t* xr = a.x + (size_t)(live ? row : 0u) * a.K;
  int8_t* cr = a.codes + (size_t)row * a.K_pad;
  for (uint32_t g = 0; g < a.G; ++g) {
    const uint32_t k0 = g * a.group;
    float amax = 0.0f;
    for (uint32_t e = lane; e < a.group; e += 64u) {
      const uint32_t k = k0 + e;
      const float v = (live && k < a.K) ? bf16_bits_to_f32(xr[k]) : 0.0f;
      amax = fmaxf(amax, fabsf(v));
    }
    amax = wave_max(amax);
    const float scale = amax > 0.0f ? amax / a.qmax : 1.0f;
    for (uint32_t e = lane; e < a.group; e += 64u) {
      const uint32_t k = k0 + e;
      const float v = (live && k < a.K) ? bf16_bits_to_f32(xr[k]) : 0.0f;
      float q = __builtin_rintf(v / scale);
      q = fminf(fmaxf(q, -a.qmax), a.qmax);
      cr[k] = (int8_t)(int)q;
    }
    if (lane == 0) a.scales[(size_t)row * a.G + g] = scale;
  }
}

// ---------------------------------------------------------------------------------------
struct GqLoraZArgs {
  const uint16_t* x;       // bf16 [M, K]
  const uint16_t* lora_a;  // bf16 [n_adapters, K, r]
  const int32_t* idx;      // int32 [M] or null (adapter 0)
  float* z;                // f32 [M, 64]
  uint32_t M, K, r, n_adapters;
};

// z[m, :] = x[m, :] @ A[idx[m]] in float32: a wave per row, lane l sums k = l, l + 64, ... in order,
// then the lanes are added by a fixed butterfly.
__global__ __launch_bounds__(256) void gq_lora_z_kernel(GqLoraZArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= a.M) return;
  int ad = a.idx ? a.idx[row] : 0;
  ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
  const uint16_t* xr = a.x + (size_t)row * a.K;
  const uint16_t* ap = a.lora_a + (size_t)ad * a.K * a.r;
  for (uint32_t r0 = 0; r0 < a.r; r0 += 8u) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (uint32_t k = lane; k < a.K; k += 64u) {
      const float xv = bf16_bits_to_f32(xr[k]);
#pragma unroll
      for (uint32_t j = 0; j < 8; ++j)
        if (r0 + j < a.r) acc[j] = fmaf(xv, bf16_bits_to_f32(ap[(size_t)k * a.r + r0 + j]), acc[j]);
    }
#pragma unroll
    for (uint32_t j = 0; j < 8; ++j) {
      float v = acc[j];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
      if (lane == 0 && r0 + j < a.r) a.z[(size_t)row * 64u + r0 + j] = v;
    }
  }
}

// ---------------------------------------------------------------------------------------
struct GqGemmArgs {
  const int8_t* codes;         // int8 [M_pad, K_pad]
  const float* xs;             // f32 [M_pad, G]
  const unsigned char* wp;     // packed weight
  const float* ws;             // f32 [G, N]
  const float* z;              // f32 [M, 64] or null
  const uint16_t* lora_b;      // bf16 [n_adapters, r, N]
  const float* lora_scaling;   // f32 [n_adapters]
  const int32_t* idx;          // int32 [M] or null
  uint16_t* out;               // bf16 [M, N]
  float* aux_base;             // f32 [M, N] base before the LoRA term, or null
  uint32_t M, N, K_pad, group, G, bits, r, n_adapters, n_col_blocks;
};

// One wave per 32 x 32 output block.  Lane l of a block holds column l % 32 and the 16 rows
// 8 (v / 4) + 4 (l / 32) + v % 4, v = 0..15.
__global__ __launch_bounds__(256) void gq_gemm_kernel(GqGemmArgs a) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t cb = blockIdx.x * 4u + wave;     // column block
  if (cb >= a.n_col_blocks) return;
  const uint32_t rb = blockIdx.y;                 // row block
  const uint32_t c = lane & 31u, h = lane >> 5;
  const uint32_t col = cb * 32u + c;
  const uint32_t kbs = a.K_pad / 32u, blocks_per_group = a.group / 32u;
  const int8_t* arow = a.codes + (size_t)(rb * 32u + c) * a.K_pad + 16u * h;
  const unsigned char* wblk = a.wp + (size_t)cb * kbs * (a.bits == 4u ? 512u : 1024u) + lane * (a.bits == 4u ? 8u : 16u);
  const bool col_ok = col < a.N;
  float outv[16];
  for (uint32_t g = 0; g < a.G; ++g) {
    v16i acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0;
    for (uint32_t b = 0; b < blocks_per_group; ++b) {
      const uint32_t kb = g * blocks_per_group + b;
      const v4i af = *reinterpret_cast<const v4i*>(arow + (size_t)kb * 32u);
      v4i bf;
      if (a.bits == 4u) {
        const uint2 raw = *reinterpret_cast<const uint2*>(wblk + (size_t)kb * 512u);
        bf[0] = (int)((raw.x << 4) & 0xf0f0f0f0u);
        bf[1] = (int)(raw.x & 0xf0f0f0f0u);
        bf[2] = (int)((raw.y << 4) & 0xf0f0f0f0u);
        bf[3] = (int)(raw.y & 0xf0f0f0f0u);
      } else {
        bf = *reinterpret_cast<const v4i*>(wblk + (size_t)kb * 1024u);
      }
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf, acc, 0, 0, 0);
    }
    const float sw = col_ok ? a.ws[(size_t)g * a.N + col] : 0.0f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const uint32_t row = rb * 32u + 8u * (v >> 2) + 4u * h + (v & 3);
      const float sx = a.xs[(size_t)row * a.G + g];
      float t = (float)acc[v] * sx;
      t = t * sw;
      if (a.bits == 4u) t = t * 0.0625f;  // exact: the codes entered as 16 * code
      outv[v] = g == 0 ? t : outv[v] + t;
    }
  }
  if (!col_ok) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const uint32_t row = rb * 32u + 8u * (v >> 2) + 4u * h + (v & 3);
    if (row >= a.M) continue;
    float y = outv[v];
    if (a.aux_base) a.aux_base[(size_t)row * a.N + col] = y;
    if (a.z) {
      int ad = a.idx ? a.idx[row] : 0;
      ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
      const float* zr = a.z + (size_t)row * 64u;
      const uint16_t* bp = a.lora_b + (size_t)ad * a.r * a.N + col;
      float low = 0.0f;
      for (uint32_t r = 0; r < a.r; ++r) low = fmaf(zr[r], bf16_bits_to_f32(bp[(size_t)r * a.N]), low);
      y = y + low * a.lora_scaling[ad];
    }
    a.out[(size_t)row * a.N + col] = (uint16_t)f32_to_bf16_bits(y);
  }
}

}  // namespace w8a8
