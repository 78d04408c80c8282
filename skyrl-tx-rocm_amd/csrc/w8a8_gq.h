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
//   gq_gemm_kernel         one wave per 64 x 64 output tile over all groups, epilogue, store
//   gq_skinny_kernel       up to 32 rows: the groups dealt to the eight waves of a column block
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
  int8_t* codes;       // matrix-core fragments [M_pad / 32][K_pad / 32][1 KiB]: lane l = row l % 32,
                       // k = 16 (l / 32) + 0..15; rows >= M and columns >= K hold zeros
  float* scales;       // f32 [G, M_pad]
  int8_t* codes_rm;    // optional row-major copy int8 [M, K_pad]
  float* scales_rm;    // optional row-major copy f32 [M, G]
  uint32_t M, M_pad, K, K_pad, group, G;
  float qmax;          // 127 or 7
  uint32_t groups_per_slice;  // grid y = slices of a row's groups (few rows: more waves per row)
};

// scale = amax > 0 ? amax / qmax : 1, code = clip(rint(x / scale), -qmax, qmax), IEEE float32
// division, round half to even (quantized_lora.py:199-212).  One wave per row, three passes over
// pieces of 8 consecutive k: the pieces' maxima go to LDS, every lane then forms the scales of its
// groups from them, and the pieces are quantized with their group's scale (K_pad <= 16384).
constexpr uint32_t kGqMaxPieces = 2048, kGqMaxGroups = 512;

__device__ inline void gq_load_piece(const GqQuantArgs& a, const uint16_t* xr, bool live, uint32_t k, float (&v)[8]) {
  if (live && k + 8u <= a.K && (a.K & 7u) == 0) {  // rows are 16-byte aligned when K % 8 == 0
    const uint4 raw = *reinterpret_cast<const uint4*>(xr + k);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (j & 1) ? __uint_as_float(w[j >> 1] & 0xffff0000u) : __uint_as_float(w[j >> 1] << 16);
  } else {
#pragma unroll
    for (uint32_t j = 0; j < 8; ++j) v[j] = (live && k + j < a.K) ? bf16_bits_to_f32(xr[k + j]) : 0.0f;
  }
}

__global__ __launch_bounds__(256) void gq_quant_kernel(GqQuantArgs a) {
  __shared__ float piece_max[4][kGqMaxPieces];
  __shared__ float group_scale[4][kGqMaxGroups];
  __shared__ float group_rscale[4][kGqMaxGroups];  // 1 / scale, or -1: divide
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t row = blockIdx.x * 4u + wave;
  if (row >= a.M_pad) return;
  const bool live = row < a.M;
  const uint16_t* xr = a.x + (size_t)(live ? row : 0u) * a.K;
  int8_t* cblk = a.codes + (size_t)(row >> 5) * (a.K_pad / 32u) * 1024u + (row & 31u) * 16u;
  const uint32_t pieces_per_group = a.group / 8u;
  const uint32_t g_lo = blockIdx.y * a.groups_per_slice;
  const uint32_t g_hi = g_lo + a.groups_per_slice < a.G ? g_lo + a.groups_per_slice : a.G;
  if (g_lo >= g_hi) return;
  const uint32_t p_lo = g_lo * pieces_per_group, n_pieces = (g_hi - g_lo) * pieces_per_group;
  auto scales_from_piece_maxima = [&]() {
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    for (uint32_t gl = lane; gl < g_hi - g_lo; gl += 64u) {
      const uint32_t g = g_lo + gl;
      float amax = 0.0f;
      for (uint32_t p = 0; p < pieces_per_group; ++p) amax = fmaxf(amax, piece_max[wave][gl * pieces_per_group + p]);
      const float scale = amax > 0.0f ? amax / a.qmax : 1.0f;
      group_scale[wave][gl] = scale;
      group_rscale[wave][gl] = (amax == amax && scale > 1e-30f && scale < 1e30f) ? __builtin_amdgcn_rcpf(scale) : -1.0f;
      a.scales[(size_t)g * a.M_pad + row] = scale;
      if (a.scales_rm && live) a.scales_rm[(size_t)row * a.G + g] = scale;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
  };
  // codes = clip(rint(v / scale)) with the correctly rounded quotient.  v * (1 / scale) with the hardware
  // reciprocal is within 3 * 2^-24 * 128 < 2.3e-5 of it (|quotient| <= qmax <= 127), and forming it biased by
  // 128 in one fused step adds at most 2^-17: both round to the same integer unless the product lies within
  // 4e-5 of a tie.  Those pieces, and groups whose scale is not an ordinary number (rscale < 0), are redone
  // with the division.  |v| <= the group's maximum, so the clip only ever acts in the redone cases.  The
  // biased value lands in its byte with one v_cvt_pk_u8_f32; flipping bit 7 makes it two's complement.
  auto quantize_piece = [&](uint32_t p, const float (&v)[8]) {
    const uint32_t k = (p_lo + p) * 8u;
    const float scale = group_scale[wave][p / pieces_per_group];
    const float rscale = group_rscale[wave][p / pieces_per_group];
    float c[8];
    float off_integer = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float t = __builtin_fmaf(v[j], rscale, 128.0f);
      c[j] = rintf(t);
      off_integer = fmaxf(off_integer, fabsf(t - c[j]));
    }
    const bool redo = rscale < 0.0f || off_integer > 0.49996f;
    if (__builtin_amdgcn_ballot_w64(redo) != 0) {  // wave-uniform
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float q = __builtin_rintf(v[j] / scale);
        q = fminf(fmaxf(q, -a.qmax), a.qmax);
        c[j] = q + 128.0f;
      }
    }
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      w[0] = __builtin_amdgcn_cvt_pk_u8_f32(c[j], (uint32_t)j, w[0]);
      w[1] = __builtin_amdgcn_cvt_pk_u8_f32(c[j + 4], (uint32_t)j, w[1]);
    }
    w[0] ^= 0x80808080u;
    w[1] ^= 0x80808080u;
    *reinterpret_cast<uint2*>(cblk + (size_t)(k >> 5) * 1024u + ((k >> 4) & 1u) * 512u + (k & 15u)) = make_uint2(w[0], w[1]);
    if (a.codes_rm && live) *reinterpret_cast<uint2*>(a.codes_rm + (size_t)row * a.K_pad + k) = make_uint2(w[0], w[1]);
  };
  if ((a.K & 7u) == 0) {
    // rows of 16-byte pieces: the wave's share of the row (at most 2048 pieces, 32 per lane) stays in registers
    // between the pass that finds the maxima and the pass that quantizes, so the row is read once
    constexpr uint32_t kIt = kGqMaxPieces / 64u;
    uint4 raw[kIt];
#pragma unroll
    for (uint32_t it = 0; it < kIt; ++it) {
      const uint32_t p = it * 64u + lane, k = (p_lo + p) * 8u;
      raw[it] = make_uint4(0u, 0u, 0u, 0u);
      if (it * 64u < n_pieces && p < n_pieces && live && k < a.K) raw[it] = *reinterpret_cast<const uint4*>(xr + k);
    }
#pragma unroll
    for (uint32_t it = 0; it < kIt; ++it) {
      const uint32_t p = it * 64u + lane;
      if (it * 64u >= n_pieces) break;  // wave-uniform
      // |bf16| compares like its 15 magnitude bits as an integer (a NaN ends above every number)
      typedef unsigned short us2 __attribute__((ext_vector_type(2)));
      us2 mx = __builtin_bit_cast(us2, raw[it].x & 0x7fff7fffu);
      mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, raw[it].y & 0x7fff7fffu));
      mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, raw[it].z & 0x7fff7fffu));
      mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, raw[it].w & 0x7fff7fffu));
      const uint32_t top = mx[0] > mx[1] ? mx[0] : mx[1];
      if (p < n_pieces) piece_max[wave][p] = __uint_as_float(top << 16);
    }
    scales_from_piece_maxima();
#pragma unroll
    for (uint32_t it = 0; it < kIt; ++it) {
      const uint32_t p = it * 64u + lane;
      if (it * 64u >= n_pieces) break;  // wave-uniform
      if (p >= n_pieces) continue;
      const uint32_t w[4] = {raw[it].x, raw[it].y, raw[it].z, raw[it].w};
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (j & 1) ? __uint_as_float(w[j >> 1] & 0xffff0000u) : __uint_as_float(w[j >> 1] << 16);
      quantize_piece(p, v);
    }
    return;
  }
  for (uint32_t p = lane; p < n_pieces; p += 64u) {
    float v[8];
    gq_load_piece(a, xr, live, (p_lo + p) * 8u, v);
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(v[j]));
    piece_max[wave][p] = m;
  }
  scales_from_piece_maxima();
  for (uint32_t p = lane; p < n_pieces; p += 64u) {
    float v[8];
    gq_load_piece(a, xr, live, (p_lo + p) * 8u, v);
    quantize_piece(p, v);
  }
}

// ---------------------------------------------------------------------------------------
struct GqLoraZArgs {
  const uint16_t* x;       // bf16 [M, K]
  const uint16_t* lora_a;  // bf16 [n_adapters, K, r]
  const int32_t* idx;      // int32 [M] or null (adapter 0)
  float* z;                // f32 [k_split][M][64]: slice s holds the sum over its range of k
  uint32_t M, K, r, n_adapters;
  uint32_t k_split, k_chunk;  // slices (grid y) and k per slice (a multiple of 64)
};

// z[m, :] = x[m, :] @ A[idx[m]] in float32: a wave per (row, k slice), lane l sums k = l, l + 64, ...
// of the slice in order for all ranks at once (RB blocks of 8 ranks in registers), then the lanes are
// added by a fixed butterfly; the consumer adds the slices in order.
template <uint32_t RB>
__global__ __launch_bounds__(256) void gq_lora_z_kernel(GqLoraZArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= a.M) return;
  int ad = a.idx ? a.idx[row] : 0;
  ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
  const uint16_t* xr = a.x + (size_t)row * a.K;
  const uint16_t* ap = a.lora_a + (size_t)ad * a.K * a.r;
  const bool vec = (a.r & 7u) == 0;  // rows of A are then 16-byte pieces
  float acc[RB * 8];
#pragma unroll
  for (uint32_t j = 0; j < RB * 8u; ++j) acc[j] = 0.0f;
  const uint32_t k_lo = blockIdx.y * a.k_chunk;
  const uint32_t k_hi = k_lo + a.k_chunk < a.K ? k_lo + a.k_chunk : a.K;
  float* zout = a.z + ((size_t)blockIdx.y * a.M + row) * 64u;
  for (uint32_t k = k_lo + lane; k < k_hi; k += 64u) {
    const float xv = bf16_bits_to_f32(xr[k]);
    const uint16_t* ar = ap + (size_t)k * a.r;
#pragma unroll
    for (uint32_t b = 0; b < RB; ++b) {
      if (b * 8u >= a.r) break;
      if (vec) {
        const uint4 raw = *reinterpret_cast<const uint4*>(ar + b * 8u);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
          const float av = (j & 1u) ? __uint_as_float(w[j >> 1] & 0xffff0000u) : __uint_as_float(w[j >> 1] << 16);
          acc[b * 8u + j] = fmaf(xv, av, acc[b * 8u + j]);
        }
      } else {
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j)
          if (b * 8u + j < a.r) acc[b * 8u + j] = fmaf(xv, bf16_bits_to_f32(ar[b * 8u + j]), acc[b * 8u + j]);
      }
    }
  }
#pragma unroll
  for (uint32_t j = 0; j < RB * 8u; ++j) {
    float v = acc[j];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    if (lane == 0 && j < a.r) zout[j] = v;
  }
}

// ---------------------------------------------------------------------------------------
struct GqGemmArgs {
  const int8_t* codes;         // fragments [M_pad / 32][K_pad / 32][1 KiB]
  const float* xs;             // f32 [G, M_pad]
  uint32_t M_pad;
  const unsigned char* wp;     // packed weight
  const float* ws;             // f32 [G, N]
  const float* z;              // f32 [rows or slots, 64] or null
  const int32_t* z_slot;       // int32 [M]: where row m's z lives (rows routed by adapter), or null: row m
  uint32_t z_slices;           // z arrives as this many K slices to add in order, z_slice_stride floats apart
  uint32_t z_slice_stride;
  const uint16_t* lora_b;      // bf16 [n_adapters, r, N]
  const float* lora_scaling;   // f32 [n_adapters]
  const int32_t* idx;          // int32 [M] or null
  uint16_t* out;               // bf16 [M, N]
  float* aux_base;             // f32 [M, N] base before the LoRA term, or null
  uint32_t M, N, K_pad, group, G, bits, r, n_adapters, n_col_blocks;
};

// One wave per 64 x 64 output tile (2 x 2 blocks of 32 x 32), four waves (128 columns) per workgroup.
// Lane l of a block holds column l % 32 and the 16 rows 8 (v / 4) + 4 (l / 32) + v % 4, v = 0..15.
// A weight fragment as it sits in memory (8 or 16 bytes per lane) and its expansion to the int8
// operand; kept apart so that a fragment loaded one step ahead is only expanded when it is used
// (expanding at load time would make the load's latency part of the step).
template <bool W4>
struct GqRawFragment { uint4 v; };

template <bool W4>
__device__ inline GqRawFragment<W4> gq_load_raw(const unsigned char* p) {
  GqRawFragment<W4> r;
  if (W4) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    r.v = make_uint4(t.x, t.y, 0u, 0u);
  } else {
    r.v = *reinterpret_cast<const uint4*>(p);
  }
  return r;
}

template <bool W4>
__device__ inline v4i gq_expand(const GqRawFragment<W4>& r) {
  v4i f;
  if (W4) {
    f[0] = (int)((r.v.x << 4) & 0xf0f0f0f0u);
    f[1] = (int)(r.v.x & 0xf0f0f0f0u);
    f[2] = (int)((r.v.y << 4) & 0xf0f0f0f0u);
    f[3] = (int)(r.v.y & 0xf0f0f0f0u);
  } else {
    f[0] = (int)r.v.x; f[1] = (int)r.v.y; f[2] = (int)r.v.z; f[3] = (int)r.v.w;
  }
  return f;
}

template <bool W4>
__device__ inline v4i gq_weight_fragment(const unsigned char* p) {
  if (W4) {
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    v4i f;
    f[0] = (int)((raw.x << 4) & 0xf0f0f0f0u);
    f[1] = (int)(raw.x & 0xf0f0f0f0u);
    f[2] = (int)((raw.y << 4) & 0xf0f0f0f0u);
    f[3] = (int)(raw.y & 0xf0f0f0f0u);
    return f;
  }
  return *reinterpret_cast<const v4i*>(p);
}

// The end of one 32-row block of a wave's tile: a row's low-rank sum scaled by its adapter's factor, the add,
// the cast, the store.  outv[j][v] is the float32 base of column block j, row 8 (v / 4) + 4 (lane / 32) + v % 4;
// lacc[j][v] the unscaled low-rank sum of the same place.
__device__ inline void gq_finish_row_block(const GqGemmArgs& a, const float (&outv)[2][16], const v16f (&lacc)[2], bool lora,
                                           uint32_t rb, const uint32_t (&col)[2], bool two_cols, uint32_t lane) {
  const uint32_t h = lane >> 5;
  float sg[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    sg[v] = 0.0f;
    if (lora) {
      const uint32_t row = rb * 32u + 8u * (v >> 2) + 4u * h + (v & 3);
      int ad = (a.idx && row < a.M) ? a.idx[row] : 0;
      ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
      sg[v] = a.lora_scaling[ad];
    }
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (j == 1 && !two_cols) break;
    if (col[j] >= a.N) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const uint32_t row = rb * 32u + 8u * (v >> 2) + 4u * h + (v & 3);
      if (row >= a.M) continue;
      float y = outv[j][v];
      if (a.aux_base) a.aux_base[(size_t)row * a.N + col[j]] = y;
      if (lora) {
        const float low = lacc[j][v] * sg[v];
        y = y + low;
      }
      a.out[(size_t)row * a.N + col[j]] = (uint16_t)f32_to_bf16_bits(y);
    }
  }
}

// Epilogue of one 32-row block of a wave's tile: the LoRA term per adapter present among the block's
// rows (their z rows staged in the wave's LDS buffer), the add, the cast, the store.  outv[j][v] is the
// float32 base of column block j, row 8 (v / 4) + 4 (lane / 32) + v % 4.
__device__ inline void gq_store_row_block(const GqGemmArgs& a, const float (&outv)[2][16], uint32_t rb,
                                          const uint32_t (&col)[2], bool two_cols, float (*zbuf)[64], uint32_t lane) {
  const bool lora = a.z != nullptr;
  v16f lacc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) lacc[j][v] = 0.0f;
  if (lora) {
    __builtin_amdgcn_wave_barrier();  // the buffer's previous use by this wave is over
    for (uint32_t t = lane; t < 32u * 64u; t += 64u) {
      const uint32_t rr = t >> 6, r = t & 63u;
      const uint32_t row = rb * 32u + rr;
      const bool ok = row < a.M && r < a.r;
      const uint32_t zrow = (ok && a.z_slot) ? (uint32_t)a.z_slot[row] : row;
      float zv = 0.0f;
      if (ok) {  // the K slices of the projection, added in order
        const float* zp = a.z + (size_t)zrow * 64u + r;
        zv = zp[0];
        for (uint32_t sl = 1; sl < a.z_slices; ++sl) zv = zv + zp[(size_t)sl * a.z_slice_stride];
      }
      zbuf[rr][r] = zv;
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    // The low-rank term on the matrix core: per 16 ranks the lane's eight z values (row lane % 32) are split
    // exactly into three bf16 terms once; every adapter present among the block's rows then takes one pass
    // in which the rows of the other adapters are zeroed, against its B values of the lane's column
    // (v_mfma_f32_32x32x16_bf16: the result lands in the layout of the integer blocks).  A row's sum is
    // scaled by its adapter's factor afterwards.
    const uint32_t rowl = lane & 31u, kg = lane >> 5;
    const uint32_t rowg = rb * 32u + rowl;
    int my_ad = -1;  // rows beyond M belong to no adapter
    if (rowg < a.M) {
      const int ad = a.idx ? a.idx[rowg] : 0;
      my_ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
    }
    for (uint32_t r0 = 0; r0 < a.r; r0 += 16u) {
      uint32_t term[3][4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        float hi[2], mid[2], lo[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const float z = zbuf[rowl][r0 + 8u * kg + 2u * (uint32_t)d + (uint32_t)e];  // (zeros beyond the rank)
          hi[e] = bf16_round_f32(z);
          const float r1 = z - hi[e];
          mid[e] = bf16_round_f32(r1);
          lo[e] = bf16_round_f32(r1 - mid[e]);
        }
        term[0][d] = pack_bf16x2(hi[0], hi[1]);
        term[1][d] = pack_bf16x2(mid[0], mid[1]);
        term[2][d] = pack_bf16x2(lo[0], lo[1]);
      }
      int done_below = -1;
      for (;;) {  // adapters present among the block's rows, smallest first (wave-uniform)
        int cand = my_ad > done_below ? my_ad : 0x7fffffff;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
          const int o = __shfl_xor(cand, off);
          cand = o < cand ? o : cand;
        }
        if (cand == 0x7fffffff) break;
        done_below = cand;
        const bool mine = my_ad == cand;
        v4i za[3];
#pragma unroll
        for (int t = 0; t < 3; ++t)
#pragma unroll
          for (int d = 0; d < 4; ++d) za[t][d] = mine ? (int)term[t][d] : 0;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (j == 1 && !two_cols) break;
          uint32_t braw[8];
#pragma unroll
          for (uint32_t e = 0; e < 8; ++e) {
            const uint32_t rank = r0 + 8u * kg + e;
            braw[e] = (col[j] < a.N && rank < a.r) ? (uint32_t)a.lora_b[((size_t)cand * a.r + rank) * a.N + col[j]] : 0u;
          }
          v4i bo;
#pragma unroll
          for (int d = 0; d < 4; ++d) bo[d] = (int)(braw[2 * d] | (braw[2 * d + 1] << 16));
#pragma unroll
          for (int t = 2; t >= 0; --t)
            lacc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, za[t]), __builtin_bit_cast(v8bf, bo),
                                                              lacc[j], 0, 0, 0);
        }
      }
    }
  }
  gq_finish_row_block(a, outv, lacc, lora, rb, col, two_cols, lane);
}

// The low-rank sums of a workgroup's 128 x 128 tile with B staged through the LDS (the stage ring is free by
// then): per 16 ranks and per batch of up to eight adapters present among the tile's rows, the four waves
// bring the adapters' B values of the tile's 128 columns in with direct-to-LDS loads (a slot of 16 ranks x
// 256 bytes per adapter, 1 KiB per instruction), and every wave then takes its passes -- one per adapter
// present in a row block, the rows of the other adapters zeroed -- with its operands from there.  Per output
// the passes, their order and their operands are those of gq_store_row_block, which asks memory for the
// same B values once per pass, row block and lane, one dependent round trip after the other.  z comes
// straight from memory: a lane's eight values of a 16-rank step are 32 consecutive bytes.
// Needs N % 8 == 0 and B aligned to 16 bytes (the 16-byte pieces), at most 64 adapters (the mask).
// LDS: [0, 32 KiB) the batch, [32 KiB, + 32) the waves' adapter masks.  All four waves must call it.
constexpr uint32_t kGqLoraLdsBytes = 32768u + 64u;
__device__ inline bool gq_tile_lora_ok(const GqGemmArgs& a) {
  return a.n_adapters <= 64u && (a.N & 7u) == 0 && (reinterpret_cast<uintptr_t>(a.lora_b) & 15u) == 0;
}
__device__ inline void gq_tile_lora_sums(const GqGemmArgs& a, unsigned char* lds, const uint32_t (&rbs)[2],
                                         const bool (&rb_ok)[2], uint32_t cbase, uint32_t wave, uint32_t wc, uint32_t lane,
                                         v16f (&lacc)[2][2]) {
  typedef __attribute__((address_space(3))) const uint16_t* lds_u16ptr;
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)lds;
  const uint32_t rowl = lane & 31u, kg = lane >> 5, c = lane & 31u;
  int my_ad[2];
  uint32_t zrow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t rowg = rbs[i] * 32u + rowl;
    my_ad[i] = -1;  // rows beyond M (and row blocks beyond the edge) belong to no adapter
    zrow[i] = 0;
    if (rb_ok[i] && rowg < a.M) {
      const int ad = a.idx ? a.idx[rowg] : 0;
      my_ad[i] = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
      zrow[i] = a.z_slot ? (uint32_t)a.z_slot[rowg] : rowg;
    }
  }
  unsigned long long pm[2] = {0ull, 0ull};  // adapters present in the wave's row blocks (wave-uniform)
  for (uint32_t ad = 0; ad < a.n_adapters; ++ad)
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (__builtin_amdgcn_ballot_w64(my_ad[i] == (int)ad) != 0) pm[i] |= 1ull << ad;
  unsigned long long* const masks = reinterpret_cast<unsigned long long*>(lds + 32768u);
  if (lane == 0) masks[wave] = pm[0] | pm[1];
  __syncthreads();
  const unsigned long long wg_mask = masks[0] | masks[1] | masks[2] | masks[3];
  // what this lane brings in per slot: rank 4 wave + lane / 16 of the step, columns 8 (lane % 16) .. + 7 of the tile
  const uint32_t ld_rank = 4u * wave + (lane >> 4), ld_col = cbase * 32u + (lane & 15u) * 8u;
  for (uint32_t r0 = 0; r0 < a.r; r0 += 16u) {
    uint32_t term[2][3][4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float z8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) z8[e] = 0.0f;
      if (my_ad[i] >= 0) {
        const float* zp = a.z + (size_t)zrow[i] * 64u + r0 + 8u * kg;
        float4 lo4 = *reinterpret_cast<const float4*>(zp), hi4 = *reinterpret_cast<const float4*>(zp + 4);
        for (uint32_t sl = 1; sl < a.z_slices; ++sl) {  // the K slices of the projection, added in order
          const float4 l2 = *reinterpret_cast<const float4*>(zp + (size_t)sl * a.z_slice_stride);
          const float4 h2 = *reinterpret_cast<const float4*>(zp + (size_t)sl * a.z_slice_stride + 4);
          lo4.x = lo4.x + l2.x; lo4.y = lo4.y + l2.y; lo4.z = lo4.z + l2.z; lo4.w = lo4.w + l2.w;
          hi4.x = hi4.x + h2.x; hi4.y = hi4.y + h2.y; hi4.z = hi4.z + h2.z; hi4.w = hi4.w + h2.w;
        }
        const float t8[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) z8[e] = r0 + 8u * kg + (uint32_t)e < a.r ? t8[e] : 0.0f;
      }
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        float hi[2], mid[2], lo[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const float z = z8[2 * d + e];
          hi[e] = bf16_round_f32(z);
          const float r1 = z - hi[e];
          mid[e] = bf16_round_f32(r1);
          lo[e] = bf16_round_f32(r1 - mid[e]);
        }
        term[i][0][d] = pack_bf16x2(hi[0], hi[1]);
        term[i][1][d] = pack_bf16x2(mid[0], mid[1]);
        term[i][2][d] = pack_bf16x2(lo[0], lo[1]);
      }
    }
    const bool ld_on = r0 + ld_rank < a.r && ld_col < a.N;
    const uint32_t ld_off = ((r0 + ld_rank) * a.N + ld_col) * 2u;
    unsigned long long rem = wg_mask;
    while (rem) {  // batches of up to eight adapters, smallest first (workgroup-uniform)
      uint32_t ads[8], nb = 0;
#pragma unroll
      for (int sl = 0; sl < 8; ++sl) {
        ads[sl] = 0;
        if (rem) {
          ads[sl] = (uint32_t)__builtin_ctzll(rem);
          rem &= rem - 1ull;
          nb = (uint32_t)sl + 1u;
        }
      }
      __syncthreads();  // the batch before has been read
#pragma unroll
      for (uint32_t sl = 0; sl < 8; ++sl) {
        if (sl < nb && ld_on)
          lds_load_1k(reinterpret_cast<const unsigned char*>(a.lora_b) + (size_t)ads[sl] * a.r * a.N * 2u, ld_off,
                      lds_addr + sl * 4096u + wave * 1024u);
      }
      wait_vmcnt<0>();
      __syncthreads();
#pragma unroll
      for (uint32_t sl = 0; sl < 8; ++sl) {
        if (sl >= nb) break;
        const uint32_t ad = ads[sl];
        if (!(((pm[0] | pm[1]) >> ad) & 1ull)) continue;  // wave-uniform
        v4i bo[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const uint32_t lcol = (2u * wc + (uint32_t)j) * 32u + c;
          const bool col_ok = cbase * 32u + lcol < a.N;
          uint32_t braw[8];
#pragma unroll
          for (uint32_t e = 0; e < 8; ++e) {
            const uint32_t rank = 8u * kg + e;
            const uint16_t v = reinterpret_cast<lds_u16ptr>((lptr_t)lds)[(sl * 16u + rank) * 128u + lcol];
            braw[e] = (col_ok && r0 + rank < a.r) ? (uint32_t)v : 0u;
          }
#pragma unroll
          for (int d = 0; d < 4; ++d) bo[j][d] = (int)(braw[2 * d] | (braw[2 * d + 1] << 16));
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          if (!((pm[i] >> ad) & 1ull)) continue;  // wave-uniform
          const bool mine = my_ad[i] == (int)ad;
          v4i za[3];
#pragma unroll
          for (int t = 0; t < 3; ++t)
#pragma unroll
            for (int d = 0; d < 4; ++d) za[t][d] = mine ? (int)term[i][t][d] : 0;
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int t = 2; t >= 0; --t)
              lacc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, za[t]),
                                                                    __builtin_bit_cast(v8bf, bo[j]), lacc[i][j], 0, 0, 0);
        }
      }
    }
  }
}

template <bool W4>
__global__ __launch_bounds__(256, 2) void gq_gemm_kernel(GqGemmArgs a) {
  __shared__ float zs[4][32][64];  // per wave: the z rows of a row block (LoRA); reads are broadcasts, no padding needed
  constexpr uint32_t kBlkBytes = W4 ? 512u : 1024u, kLaneBytes = W4 ? 8u : 16u;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t cb0 = (blockIdx.x * 4u + wave) * 2u;  // first of the wave's two column blocks
  const uint32_t rb0 = blockIdx.y * 2u;                // first of its two row blocks
  const bool active = cb0 < a.n_col_blocks;            // idle waves still reach the barrier-free end
  if (!active) return;
  const uint32_t c = lane & 31u, h = lane >> 5;
  const uint32_t kbs = a.K_pad / 32u, blocks_per_group = a.group / 32u;
  const uint32_t n_rb = (a.M + 31u) / 32u;
  // a tile that hangs over the edge re-reads its last valid block; those results are never stored
  const uint32_t rb1 = rb0 + 1u < n_rb ? rb0 + 1u : rb0;
  const uint32_t cb1 = cb0 + 1u < a.n_col_blocks ? cb0 + 1u : cb0;
  const int8_t* ar0 = a.codes + (size_t)rb0 * kbs * 1024u + lane * 16u;
  const int8_t* ar1 = a.codes + (size_t)rb1 * kbs * 1024u + lane * 16u;
  const unsigned char* w0 = a.wp + (size_t)cb0 * kbs * kBlkBytes + lane * kLaneBytes;
  const unsigned char* w1 = a.wp + (size_t)cb1 * kbs * kBlkBytes + lane * kLaneBytes;
  const uint32_t col[2] = {cb0 * 32u + c, cb1 * 32u + c};
  const uint32_t rbs[2] = {rb0, rb1};
  float outv[2][2][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) outv[i][j][v] = 0.0f;
  v16i acc[2][2];
  float sw[2];
  float4 sx4[2][4];
  // the group's scales are requested when it starts so that they have arrived when its MFMAs end
  auto load_scales = [&](uint32_t g) {
#pragma unroll
    for (int j = 0; j < 2; ++j) sw[j] = col[j] < a.N ? a.ws[(size_t)g * a.N + col[j]] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q)  // rows 8 q + 4 h + 0..3 of the block: four consecutive scales
        sx4[i][q] = *reinterpret_cast<const float4*>(a.xs + (size_t)g * a.M_pad + rbs[i] * 32u + 8u * q + 4u * h);
  };
  // one k block: four MFMAs (from zero when the block opens a group) and, when it closes a group,
  // (f32(acc) * sx) * sw added in group order; for 4-bit codes sw carries the exact factor 1/16
  auto step = [&](uint32_t kb, const v4i& fa0, const v4i& fa1, const GqRawFragment<W4>& r0, const GqRawFragment<W4>& r1) {
    const v4i fb0 = gq_expand<W4>(r0), fb1 = gq_expand<W4>(r1);
    if (kb % blocks_per_group == 0) {
      const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb0, zero, 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb1, zero, 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb0, zero, 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb1, zero, 0, 0, 0);
    } else {
      acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb1, acc[1][1], 0, 0, 0);
    }
    if ((kb + 1u) % blocks_per_group == 0) {
      float swl[2] = {sw[0], sw[1]};
      if (W4) {
        swl[0] = swl[0] * 0.0625f;
        swl[1] = swl[1] * 0.0625f;
      }
      float4 sxl[2][4];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) sxl[i][q] = sx4[i][q];
      const uint32_t gn = (kb + 1u) / blocks_per_group;
      if (gn < a.G) load_scales(gn);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float sxq[4] = {sxl[i][q].x, sxl[i][q].y, sxl[i][q].z, sxl[i][q].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int v = 4 * q + e;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              float t = (float)acc[i][j][v] * sxq[e];
              t = t * swl[j];
              outv[i][j][v] = outv[i][j][v] + t;  // from +0: the first term as it is (a product is never -0 here)
            }
          }
        }
    }
  };
  // two sets of fragments take turns: one is used while the other travels (no copies between steps:
  // the loop is unrolled by the number of sets so that every set has its own registers; four sets
  // were measured slower)
  constexpr uint32_t kSets = 2;
  v4i fa[kSets][2];
  GqRawFragment<W4> fr[kSets][2];
  auto load_set = [&](uint32_t set, uint32_t kb) {
    const uint32_t k = kb < kbs ? kb : kbs - 1u;  // beyond the end: a repeated block, unused
    fa[set][0] = *reinterpret_cast<const v4i*>(ar0 + (size_t)k * 1024u);
    fa[set][1] = *reinterpret_cast<const v4i*>(ar1 + (size_t)k * 1024u);
    fr[set][0] = gq_load_raw<W4>(w0 + (size_t)k * kBlkBytes);
    fr[set][1] = gq_load_raw<W4>(w1 + (size_t)k * kBlkBytes);
  };
#pragma unroll
  for (uint32_t u = 0; u + 1u < kSets; ++u) load_set(u, u);
  load_scales(0);
  for (uint32_t kb = 0; kb < kbs; kb += kSets) {
#pragma unroll
    for (uint32_t u = 0; u < kSets; ++u) {
      load_set((u + kSets - 1u) % kSets, kb + u + kSets - 1u);
      if (kb + u < kbs) step(kb + u, fa[u][0], fa[u][1], fr[u][0], fr[u][1]);
    }
  }
  // ---- epilogue: LoRA term per adapter present in the tile, store
  gq_store_row_block(a, outv[0], rb0, col, cb1 != cb0, zs[wave], lane);
  if (rb1 != rb0) gq_store_row_block(a, outv[1], rb1, col, cb1 != cb0, zs[wave], lane);
}

// ---------------------------------------------------------------------------------------
// The same product for groups that are multiples of 64 k, staged through the LDS: a workgroup of four
// waves (2 x 2) owns a 128 x 128 output tile; per 64-wide k step its activation fragments (8 KiB), weight
// fragments (4 or 8 KiB) and the group's scales (128 column and 128 row scales) arrive once per workgroup by
// direct-to-LDS loads, three steps ahead, and every wave reads the fragments of its 64 x 64 share from
// there.  Per output the arithmetic and its order are those of gq_gemm_kernel (the step and the epilogue
// are shared), so the two kernels agree bit for bit; this one asks the L2 for half the bytes and keeps
// three steps in flight instead of one.
constexpr uint32_t kGqLdsStages = 4;
__host__ __device__ constexpr uint32_t gq_lds_stage_bytes(bool w4) { return 8192u + (w4 ? 4096u : 8192u) + 1024u; }
__host__ __device__ constexpr uint32_t gq_lds_bytes(bool w4) { return kGqLdsStages * gq_lds_stage_bytes(w4); }
static_assert(gq_lds_bytes(true) >= kGqLoraLdsBytes && gq_lds_bytes(true) >= 4u * 32u * 64u * 4u, "the epilogue reuses the ring");

template <bool W4>
__global__ __launch_bounds__(256, 2) void gq_gemm_lds_kernel(GqGemmArgs a) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char gq_lds[];  // the stage ring; the epilogue's z rows afterwards
  constexpr uint32_t kStage = gq_lds_stage_bytes(W4), kWOff = 8192u, kSOff = 8192u + (W4 ? 4096u : 8192u);
  constexpr uint32_t kWBlk = W4 ? 512u : 1024u;      // bytes of a weight fragment (one column block, one k block)
  constexpr uint32_t kLoads = 2u + (W4 ? 1u : 2u) + 1u;  // direct-to-LDS loads per wave and stage
  constexpr uint32_t NS = kGqLdsStages;
  typedef __attribute__((address_space(3))) const unsigned char* lds_cptr;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wr = wave >> 1, wc = wave & 1u;
  const uint32_t c = lane & 31u, h = lane >> 5;
  const uint32_t kbs = a.K_pad / 32u, blocks_per_group = a.group / 32u;  // both even here
  const uint32_t n_stages = kbs / 2u;
  const uint32_t n_rb = a.M_pad / 32u;
  const uint32_t rbase = blockIdx.y * 4u, cbase = blockIdx.x * 4u;
  // blocks that hang over the edge are read from the last valid one; their results are never stored
  auto rb_of = [&](uint32_t l) { return rbase + l < n_rb ? rbase + l : n_rb - 1u; };
  auto cb_of = [&](uint32_t l) { return cbase + l < a.n_col_blocks ? cbase + l : a.n_col_blocks - 1u; };
  const uint32_t rbs[2] = {rb_of(2u * wr), rb_of(2u * wr + 1u)};
  const uint32_t cbs[2] = {cb_of(2u * wc), cb_of(2u * wc + 1u)};
  const uint32_t col[2] = {cbs[0] * 32u + c, cbs[1] * 32u + c};
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)gq_lds;
  // what this wave brings in per stage: row block `wave` (2 KiB), column block `wave` (1 or 2 KiB), 64 scales
  const unsigned char* const a_src = reinterpret_cast<const unsigned char*>(a.codes) + (size_t)rb_of(wave) * kbs * 1024u;
  const unsigned char* const w_src = a.wp + (size_t)cb_of(wave) * kbs * kWBlk;
  uint32_t s_idx;  // the wave's scale of a group: a column (waves 0, 1) or a row (waves 2, 3), clamped to the last one
  if (wave < 2u) {
    const uint32_t cc = cbase * 32u + wave * 64u + lane;
    s_idx = cc < a.N ? cc : a.N - 1u;
  } else {
    const uint32_t rr = rbase * 32u + (wave - 2u) * 64u + lane;
    s_idx = rr < a.M_pad ? rr : a.M_pad - 1u;
  }
  const uint32_t stages_per_group = blocks_per_group / 2u;
  const float* const s_src = wave < 2u ? a.ws : a.xs;     // the wave's scales: one row of them per group
  const uint32_t s_stride = wave < 2u ? a.N : a.M_pad;
  uint32_t ld_sig = 0, ld_group = 0;                      // stage inside its group and group of the next stage requested
  auto load_stage = [&](uint32_t st) {
    const uint32_t slot = lds0 + (st % NS) * kStage;
    lds_load_1k(a_src + (size_t)st * 2048u, lane * 16u, slot + wave * 2048u);
    lds_load_1k(a_src + (size_t)st * 2048u, 1024u + lane * 16u, slot + wave * 2048u + 1024u);
    lds_load_1k(w_src + (size_t)st * 2u * kWBlk, lane * 16u, slot + kWOff + wave * 2u * kWBlk);
    if (!W4) lds_load_1k(w_src + (size_t)st * 2u * kWBlk, 1024u + lane * 16u, slot + kWOff + wave * 2u * kWBlk + 1024u);
    lds_gather_dword(s_src + (size_t)ld_group * s_stride, s_idx * 4u, slot + kSOff + wave * 256u);
    if (++ld_sig == stages_per_group) { ld_sig = 0; ++ld_group; }  // (stages are requested in order)
  };

  float outv[2][2][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) outv[i][j][v] = 0.0f;
  v16i acc[2][2];
  // one k block, as in gq_gemm_kernel: four MFMAs (from zero when the block opens a group) and, when it
  // closes a group, (f32(acc) * sx) * sw added in group order; for 4-bit codes sw carries the exact 1/16
  // (opens / closes: whether the k block is the first / last of its group, workgroup-uniform and kept by
  // counting: a remainder per k block costs more instructions than the block's four MFMAs leave room for)
  auto step = [&](bool opens, bool closes, const v4i& fa0, const v4i& fa1, const GqRawFragment<W4>& r0,
                  const GqRawFragment<W4>& r1, lds_cptr sc) {
    const v4i fb0 = gq_expand<W4>(r0), fb1 = gq_expand<W4>(r1);
    if (opens) {
      const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb0, zero, 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb1, zero, 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb0, zero, 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb1, zero, 0, 0, 0);
    } else {
      acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa0, fb1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1, fb1, acc[1][1], 0, 0, 0);
    }
    if (closes) {
      typedef __attribute__((address_space(3))) const float* lds_fptr;
      typedef float gq_f4 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) const gq_f4* lds_f4ptr;
      float swl[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        swl[j] = reinterpret_cast<lds_fptr>(sc)[(2u * wc + (uint32_t)j) * 32u + c];
        if (W4) swl[j] = swl[j] * 0.0625f;
      }
      // a fragment's sixteen sums at a time, each of the four steps for all sixteen before the next step (the
      // same operations per output; measured 3 % faster than output by output, where every instruction
      // needs the result of the one in front of it)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        gq_f4 s4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          s4[q] = *reinterpret_cast<lds_f4ptr>(sc + 512u + ((2u * wr + (uint32_t)i) * 32u + 8u * q + 4u * h) * 4u);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float t[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) t[v] = (float)acc[i][j][v];
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int v = 0; v < 16; ++v) t[v] = t[v] * s4[v >> 2][v & 3];
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int v = 0; v < 16; ++v) t[v] = t[v] * swl[j];
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int v = 0; v < 16; ++v) outv[i][j][v] = outv[i][j][v] + t[v];
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };

  for (uint32_t st = 0; st + 1u < NS && st < n_stages; ++st) load_stage(st);
  uint32_t sig = 0;  // stage inside its group
  for (uint32_t st = 0; st < n_stages; ++st) {
    // stage st has landed once at most the NS - 2 younger stages are outstanding (none are issued near the end)
    if (st + NS - 2u < n_stages) wait_vmcnt<(NS - 2) * kLoads>();
    else wait_vmcnt<0>();
    lds_barrier();  // everybody's pieces of stage st; and every wave is done with stage st - 1
    if (st + NS - 1u < n_stages) load_stage(st + NS - 1u);  // into the slot of stage st - 1
    lds_cptr slot = reinterpret_cast<lds_cptr>((uintptr_t)(lds0 + (st % NS) * kStage));
    v4i fa[2][2];
    GqRawFragment<W4> fr[2][2];
#pragma unroll
    for (uint32_t kl = 0; kl < 2; ++kl) {
#pragma unroll
      for (uint32_t i = 0; i < 2; ++i) {
        typedef __attribute__((address_space(3))) const v4i* lds_v4ptr;
        fa[kl][i] = *reinterpret_cast<lds_v4ptr>(slot + (2u * wr + i) * 2048u + kl * 1024u + lane * 16u);
        lds_cptr wp = slot + kWOff + (2u * wc + i) * 2u * kWBlk + kl * kWBlk + lane * (W4 ? 8u : 16u);
        if (W4) {
          typedef uint32_t gq_u2 __attribute__((ext_vector_type(2)));
          typedef __attribute__((address_space(3))) const gq_u2* lds_u2ptr;
          const gq_u2 t = *reinterpret_cast<lds_u2ptr>(wp);
          fr[kl][i].v = make_uint4(t[0], t[1], 0u, 0u);
        } else {
          typedef uint32_t gq_u4 __attribute__((ext_vector_type(4)));
          typedef __attribute__((address_space(3))) const gq_u4* lds_u4ptr;
          const gq_u4 t = *reinterpret_cast<lds_u4ptr>(wp);
          fr[kl][i].v = make_uint4(t[0], t[1], t[2], t[3]);
        }
      }
    }
    const bool last_of_group = sig + 1u == stages_per_group;
    step(sig == 0u, false, fa[0][0], fa[0][1], fr[0][0], fr[0][1], slot + kSOff);
    step(false, last_of_group, fa[1][0], fa[1][1], fr[1][0], fr[1][1], slot + kSOff);
    sig = last_of_group ? 0u : sig + 1u;
  }
  // ---- epilogue: LoRA term per adapter present in the tile, store (the ring is free: its last reads are done)
  lds_barrier();
  const bool two_cols = cbase + 2u * wc + 1u < a.n_col_blocks;
  const bool rb_ok[2] = {rbase + 2u * wr < n_rb, rbase + 2u * wr + 1u < n_rb};
  const bool cols_ok = cbase + 2u * wc < a.n_col_blocks;
  if (a.z && gq_tile_lora_ok(a)) {  // workgroup-uniform
    v16f lacc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) lacc[i][j][v] = 0.0f;
    gq_tile_lora_sums(a, gq_lds, rbs, rb_ok, cbase, wave, wc, lane, lacc);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (rb_ok[i] && cols_ok) gq_finish_row_block(a, outv[i], lacc[i], true, rbs[i], col, two_cols, lane);
    return;
  }
  float (*zs)[64] = reinterpret_cast<float (*)[64]>(gq_lds + wave * 32u * 64u * 4u);
  if (rb_ok[0] && cols_ok) {
    gq_store_row_block(a, outv[0], rbs[0], col, two_cols, zs, lane);
    if (rb_ok[1]) gq_store_row_block(a, outv[1], rbs[1], col, two_cols, zs, lane);
  }
}

// ---------------------------------------------------------------------------------------
// Up to 32 rows (decode): a workgroup of eight waves owns one 32-column block for all of K.  Wave w
// takes a contiguous range of groups, streams its weight fragments eight k blocks ahead, forms its
// groups' float32 terms in group order, and the eight partial sums are added in wave order through
// LDS -- the groups are summed in order inside a wave and the waves in order, which differs from
// the strictly sequential float32 sum of the reference only in rounding (inside the bf16 tolerance;
// the result is the same from run to run).
constexpr uint32_t kGqSkinnyWaves = 8;

template <bool W4>
__global__ __launch_bounds__(512) void gq_skinny_kernel(GqGemmArgs a) {
  __shared__ float red[kGqSkinnyWaves][16][64];
  constexpr uint32_t kBlkBytes = W4 ? 512u : 1024u, kLaneBytes = W4 ? 8u : 16u, U = 8u;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t cb = blockIdx.x;
  const uint32_t c = lane & 31u, h = lane >> 5;
  const uint32_t col = cb * 32u + c;
  const uint32_t kbs = a.K_pad / 32u, bpg = a.group / 32u;
  const uint32_t g_lo = (wave * a.G) / kGqSkinnyWaves, g_hi = ((wave + 1u) * a.G) / kGqSkinnyWaves;
  const int8_t* ap = a.codes + lane * 16u;  // row block 0
  const unsigned char* wp = a.wp + (size_t)cb * kbs * kBlkBytes + lane * kLaneBytes;
  float part[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) part[v] = 0.0f;
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  const uint32_t kb_lo = g_lo * bpg, kb_hi = g_hi * bpg;
  // the scales of the group in progress, requested a group ahead
  auto load_scales = [&](uint32_t g, float& sw, float4 (&sx)[4]) {
    const uint32_t gg = g < a.G ? g : a.G - 1u;
    sw = col < a.N ? a.ws[(size_t)gg * a.N + col] : 0.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q) sx[q] = *reinterpret_cast<const float4*>(a.xs + (size_t)gg * a.M_pad + 8u * q + 4u * h);
  };
  float sw_cur;
  float4 sx_cur[4];
  load_scales(g_lo, sw_cur, sx_cur);
  bool first = true;
  for (uint32_t base = kb_lo; base < kb_hi; base += U) {
    v4i fa[U], fb[U];
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t kb = base + u < kb_hi ? base + u : kb_hi - 1u;  // the tail repeats a block, unused
      fa[u] = *reinterpret_cast<const v4i*>(ap + (size_t)kb * 1024u);
      fb[u] = gq_weight_fragment<W4>(wp + (size_t)kb * kBlkBytes);
    }
#pragma unroll
    for (uint32_t u = 0; u < U; ++u) {
      const uint32_t kb = base + u;
      if (kb < kb_hi) {  // wave-uniform
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[u], fb[u], acc, 0, 0, 0);
        if ((kb + 1u) % bpg == 0) {  // the group is complete
          float sw = sw_cur;
          if (W4) sw = sw * 0.0625f;
          float4 sx[4] = {sx_cur[0], sx_cur[1], sx_cur[2], sx_cur[3]};
          load_scales((kb + 1u) / bpg, sw_cur, sx_cur);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float sxq[4] = {sx[q].x, sx[q].y, sx[q].z, sx[q].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int v = 4 * q + e;
              float t = (float)acc[v] * sxq[e];
              t = t * sw;
              part[v] = first ? t : part[v] + t;
              acc[v] = 0;
            }
          }
          first = false;
        }
      }
    }
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) red[wave][v][lane] = part[v];
  __shared__ float zsum[32][64];
  if (a.z) {
    for (uint32_t q = tid; q < 32u * 64u; q += 512u) {
      const uint32_t row = q >> 6, r = q & 63u;
      float zv = 0.0f;
      if (row < a.M && r < a.r) {
        const float* zp = a.z + (size_t)(a.z_slot ? (uint32_t)a.z_slot[row] : row) * 64u + r;
        for (uint32_t sl = 0; sl < a.z_slices; ++sl) zv = sl == 0 ? zp[0] : zv + zp[(size_t)sl * a.z_slice_stride];
      }
      zsum[row][r] = zv;
    }
  }
  __syncthreads();
  for (uint32_t o = tid; o < 1024u; o += 512u) {
    const uint32_t v = o >> 6, l = o & 63u;
    const uint32_t row = 8u * (v >> 2) + 4u * (l >> 5) + (v & 3u), ocol = cb * 32u + (l & 31u);
    if (row >= a.M || ocol >= a.N) continue;
    float y = 0.0f;
    bool any = false;
#pragma unroll
    for (uint32_t w = 0; w < kGqSkinnyWaves; ++w) {
      const bool has = (w * a.G) / kGqSkinnyWaves < ((w + 1u) * a.G) / kGqSkinnyWaves;  // the wave had groups
      if (has) {
        y = any ? y + red[w][v][l] : red[w][v][l];
        any = true;
      }
    }
    if (a.aux_base) a.aux_base[(size_t)row * a.N + ocol] = y;
    if (a.z) {
      int ad = a.idx ? a.idx[row] : 0;
      ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
      const float* zr = zsum[row];
      const uint16_t* bp = a.lora_b + (size_t)ad * a.r * a.N + ocol;
      float low = 0.0f;
      for (uint32_t r0 = 0; r0 < a.r; r0 += 8u) {
        uint16_t braw[8];
#pragma unroll
        for (uint32_t t = 0; t < 8; ++t) braw[t] = r0 + t < a.r ? bp[(size_t)(r0 + t) * a.N] : (uint16_t)0;
#pragma unroll
        for (uint32_t t = 0; t < 8; ++t)
          if (r0 + t < a.r) low = fmaf(zr[r0 + t], bf16_bits_to_f32(braw[t]), low);
      }
      y = y + low * a.lora_scaling[ad];
    }
    a.out[(size_t)row * a.N + ocol] = (uint16_t)f32_to_bf16_bits(y);
  }
}

}  // namespace w8a8
