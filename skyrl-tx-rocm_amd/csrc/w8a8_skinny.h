// Skinny-M (decode) path, M <= 32 rows: the weight is streamed exactly once from HBM.
//   1. skinny_quant_kernel   one workgroup per row: (RMSNorm,) absmax, scale, int8 codes in
//                            MFMA operand order.
//   2. skinny_stream_kernel  work units of two kinds share one launch:
//        - weight units: a wave owns 32 output columns x a K range, loads 1 KiB weight blocks
//          straight from HBM into MFMA operands (no LDS: every block is used once), the four
//          waves of a workgroup are reduced through LDS and stored as an int32 partial;
//        - LoRA-A units: z_part[chunk][m][:] = x[m, chunk] @ A[idx[m]][chunk, :] in float32.
//   3. skinny_epilogue_kernel  sums the int32 partials (exact, order-free) and the float32 z
//                            partials (fixed order), applies (float(acc) * sx) * sw
//                            + s * (z @ B[idx[m]]) + residual and casts to bf16 once.
// No atomics: results are bit-identical from run to run.
#pragma once
#include "../../include/mi355_w8a8.h"
#include "w8a8_device.h"

namespace w8a8 {

constexpr int kSkinnyMaxRows = 32;
constexpr uint32_t kSkinnyMaxKSplit = 8;
constexpr uint32_t kSkinnyMaxZChunks = 64;
constexpr uint32_t kSkinnyZChunkK = 512;  // K elements per LoRA-A work unit (per row)

struct SkinnyLayout {
  uint64_t acc_part, z_part, total;
  uint32_t ksplit, kb_per_wave, z_chunks, z_chunk_k;
};

inline SkinnyLayout skinny_layout(uint32_t m, uint32_t k, uint32_t n) {
  (void)m;
  SkinnyLayout L{};
  const uint32_t KB = k_padded(k) / 32u;
  const uint32_t nb = (n + 31u) / 32u;
  // enough workgroups for ~3 per CU, at least 4 k-blocks per wave
  uint32_t ks = (768u + nb - 1u) / nb;
  if (ks < 1u) ks = 1u;
  if (ks > kSkinnyMaxKSplit) ks = kSkinnyMaxKSplit;
  while (ks > 1u && KB / (ks * 4u) < 4u) --ks;
  L.ksplit = ks;
  L.kb_per_wave = (KB + ks * 4u - 1u) / (ks * 4u);
  uint32_t zc = (k + kSkinnyZChunkK - 1u) / kSkinnyZChunkK;
  uint32_t zk = kSkinnyZChunkK;
  while (zc > kSkinnyMaxZChunks) { zk *= 2u; zc = (k + zk - 1u) / zk; }
  L.z_chunks = zc;
  L.z_chunk_k = zk;
  L.acc_part = 0;
  uint64_t off = (uint64_t)kSkinnyMaxKSplit * kSkinnyMaxRows * n_padded(n) * 4u;
  L.z_part = off;
  off += (uint64_t)kSkinnyMaxZChunks * kSkinnyMaxRows * kMaxRank * 4u;
  L.total = off;
  return L;
}

inline uint64_t skinny_workspace_bytes(uint32_t m, uint32_t n) {
  (void)m;
  return (uint64_t)kSkinnyMaxKSplit * kSkinnyMaxRows * n_padded(n) * 4u +
         (uint64_t)kSkinnyMaxZChunks * kSkinnyMaxRows * kMaxRank * 4u;
}
inline bool skinny_supported() { return true; }

// ---------------------------------------------------------------------------------------
struct SkinnyQuantArgs {
  const uint16_t* x;     // bf16 [M, K]
  const float* gamma;    // f32 [K] or null
  float eps;
  uint32_t M, K, K_pad, KB;
  unsigned char* xq;     // packed codes, one 32-row block [KB][1 KiB]
  float* sx;             // f32 [32]
  int8_t* codes_rm;      // optional row-major copy
  float* scales_rm;      // optional
  uint16_t* xn;          // bf16 [M, K] normalized rows (RMSNorm only) or null
  uint16_t* xn_aux;      // optional copy for the caller
  // LoRA-A work units that share the launch (they need only x, not the codes); with RMSNorm they
  // would need the normalized rows, so then they run in the stream kernel instead
  const uint16_t* lora_a;  // bf16 [n_adapters, K, r] or null
  const int32_t* idx;      // adapter per row or null
  float* z_part;           // f32 [z_chunks][32][kMaxRank]
  uint32_t n_adapters, r, z_chunks, z_chunk_k, n_z_units;
};

// z_part[ch][m][:] = x[m, chunk ch] @ A[idx[m]][chunk ch, :] in float32.  Thread (kl, q)
// accumulates rank columns 8q..8q+7 over the rows k = k_begin + kl + kpt*j; lanes with equal q are
// reduced by a fixed butterfly and the waves are added in wave order.
template <int THREADS>
__device__ inline void skinny_lora_a_unit(const uint16_t* __restrict__ xsrc, const uint16_t* __restrict__ lora_a,
                                          const int32_t* __restrict__ idx, float* __restrict__ z_part,
                                          uint32_t unit, uint32_t K, uint32_t n_adapters, uint32_t r,
                                          uint32_t z_chunks, uint32_t z_chunk_k, float (*zw)[64]) {
  constexpr uint32_t kWaves = THREADS / 64;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t m = unit / z_chunks, ch = unit % z_chunks;
  int ad = idx ? idx[m] : 0;
  ad = ad < 0 ? 0 : (ad >= (int)n_adapters ? (int)n_adapters - 1 : ad);
  const uint16_t* Ar = lora_a + (size_t)ad * K * r;
  const uint16_t* xr = xsrc + (size_t)m * K;
  const uint32_t rch = (r + 7u) / 8u;  // 8-wide rank chunks
  const uint32_t rch2 = rch <= 1u ? 1u : (rch <= 2u ? 2u : (rch <= 4u ? 4u : 8u));
  const uint32_t kpt = THREADS / rch2;
  const uint32_t q = tid % rch2, kl = tid / rch2;
  float accz[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const uint32_t k_begin = ch * z_chunk_k;
  uint32_t k_end = k_begin + z_chunk_k;
  if (k_end > K) k_end = K;
  if (q < rch) {
    for (uint32_t k = k_begin + kl; k < k_end; k += kpt) {
      const float xv = bf16_bits_to_f32(xr[k]);
      const uint16_t* src = Ar + (size_t)k * r + q * 8u;
      if ((r & 7u) == 0) {
        const v8us w = *reinterpret_cast<const v8us*>(src);
#pragma unroll
        for (int e = 0; e < 8; ++e) accz[e] = fmaf(xv, bf16_bits_to_f32(w[e]), accz[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (q * 8u + e < r) accz[e] = fmaf(xv, bf16_bits_to_f32(src[e]), accz[e]);
      }
    }
  }
  for (uint32_t off = rch2; off < 64u; off <<= 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) accz[e] += __shfl_xor(accz[e], (int)off, 64);
  }
  if (lane < rch2) {
#pragma unroll
    for (int e = 0; e < 8; ++e) zw[wave][lane * 8u + e] = accz[e];
  }
  __syncthreads();
  if (tid < (uint32_t)kMaxRank) {
    float sum = zw[0][tid];
#pragma unroll
    for (uint32_t w = 1; w < kWaves; ++w) sum += zw[w][tid];
    z_part[((size_t)ch * kSkinnyMaxRows + m) * kMaxRank + tid] = (tid < r) ? sum : 0.f;
  }
}

template <bool RMS>
__global__ __launch_bounds__(1024) void skinny_quant_kernel(SkinnyQuantArgs a) {
  __shared__ float red_max[16];
  __shared__ double red_sum[16];
  __shared__ float zw[16][64];
  if (blockIdx.x >= a.M) {
    skinny_lora_a_unit<1024>(a.x, a.lora_a, a.idx, a.z_part, blockIdx.x - a.M, a.K, a.n_adapters, a.r,
                             a.z_chunks, a.z_chunk_k, zw);
    return;
  }
  const uint32_t m = blockIdx.x;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint16_t* xr = a.x + (size_t)m * a.K;
  float v[2][8];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t k0 = (j * 1024u + tid) * 8u;
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (k0 < a.K) raw = *reinterpret_cast<const uint4*>(xr + k0);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[j][2 * e] = __uint_as_float(w[e] << 16);
      v[j][2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  }
  if (RMS) {
    double ss = 0.0;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += (double)v[j][e] * (double)v[j][e];
    ss = wave_sum(ss);
    if (lane == 0) red_sum[wave] = ss;
    __syncthreads();
    double tot = 0.0;
#pragma unroll
    for (int w = 0; w < 16; ++w) tot += red_sum[w];
    const float var = (float)(tot / (double)a.K);
    const float inv = 1.0f / sqrtf(var + a.eps);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t k0 = (j * 1024u + tid) * 8u;
      if (k0 < a.K) {
        const float4 g0 = *reinterpret_cast<const float4*>(a.gamma + k0);
        const float4 g1 = *reinterpret_cast<const float4*>(a.gamma + k0 + 4);
        const float gm[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        uint32_t packed[4];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float t = v[j][e] * inv;
          t = t * gm[e];
          const uint32_t b = f32_to_bf16_bits(t);
          v[j][e] = __uint_as_float(b << 16);
          if (e & 1) packed[e >> 1] |= b << 16; else packed[e >> 1] = b;
        }
        const uint4 o = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        if (a.xn) *reinterpret_cast<uint4*>(a.xn + (size_t)m * a.K + k0) = o;
        if (a.xn_aux) *reinterpret_cast<uint4*>(a.xn_aux + (size_t)m * a.K + k0) = o;
      }
    }
  }
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[j][e]));
  amax = wave_max(amax);
  if (lane == 0) red_max[wave] = amax;
  __syncthreads();
  amax = 0.0f;
#pragma unroll
  for (int w = 0; w < 16; ++w) amax = fmaxf(amax, red_max[w]);
  const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
  if (tid == 0) {
    a.sx[m] = scale;
    if (a.scales_rm) a.scales_rm[m] = scale;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t k0 = (j * 1024u + tid) * 8u;
    if (k0 >= a.K_pad) continue;
    uint32_t lo = 0, hi = 0;
    if (k0 < a.K) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float q = rintf(v[j][e] / scale);
        q = fminf(fmaxf(q, -127.0f), 127.0f);
        const uint32_t b = (uint32_t)(int)q & 0xffu;
        if (e < 4) lo |= b << (8 * e); else hi |= b << (8 * (e - 4));
      }
      if (a.codes_rm) *reinterpret_cast<uint2*>(a.codes_rm + (size_t)m * a.K + k0) = make_uint2(lo, hi);
    }
    *reinterpret_cast<uint2*>(a.xq + packed_offset(m, k0, a.KB)) = make_uint2(lo, hi);
  }
}

// ---------------------------------------------------------------------------------------
struct SkinnyStreamArgs {
  const unsigned char* xq;   // packed codes of the single 32-row block
  const unsigned char* wp;   // packed weight
  int32_t* acc_part;         // int32 [ksplit][32][Nb*32]
  const uint16_t* xsrc;      // bf16 [M, K] rows for LoRA-A (x or normalized rows) or null
  const uint16_t* lora_a;    // bf16 [n_adapters, K, r]
  const int32_t* idx;        // adapter per row or null
  float* z_part;             // f32 [z_chunks][32][kMaxRank]
  uint32_t M, K, KB, NB, ksplit, kb_per_wave, n_adapters, r, z_chunks, z_chunk_k, n_z_units;
};

__global__ __launch_bounds__(256) void skinny_stream_kernel(SkinnyStreamArgs a) {
  __shared__ __attribute__((aligned(16))) int red[3][16][64];
  __shared__ float zw[4][64];
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (blockIdx.x < a.n_z_units) {
    skinny_lora_a_unit<256>(a.xsrc, a.lora_a, a.idx, a.z_part, blockIdx.x, a.K, a.n_adapters, a.r,
                            a.z_chunks, a.z_chunk_k, zw);
    return;
  }
  // ---- weight unit: column block nb, K split ks; wave w takes k-blocks [kb0, kb1)
  const uint32_t u = blockIdx.x - a.n_z_units;
  const uint32_t nb = u % a.NB, ks = u / a.NB;
  uint32_t kb0 = (ks * 4u + wave) * a.kb_per_wave, kb1 = kb0 + a.kb_per_wave;
  if (kb1 > a.KB) kb1 = a.KB;
  const unsigned char* wsrc = a.wp + (size_t)nb * a.KB * kBlockBytes + lane * 16u;
  const unsigned char* xsrc = a.xq + lane * 16u;
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  uint32_t kb = kb0;
  for (; kb + 8u <= kb1; kb += 8u) {
    v4i wf[8], xf[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      wf[t] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wsrc + (size_t)(kb + t) * kBlockBytes));
      xf[t] = *reinterpret_cast<const v4i*>(xsrc + (size_t)(kb + t) * kBlockBytes);
    }
#pragma unroll
    for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[t], wf[t], acc, 0, 0, 0);
  }
  for (; kb < kb1; ++kb) {
    const v4i wf = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wsrc + (size_t)kb * kBlockBytes));
    const v4i xf = *reinterpret_cast<const v4i*>(xsrc + (size_t)kb * kBlockBytes);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf, wf, acc, 0, 0, 0);
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) red[wave - 1][e][lane] = acc[e];
  }
  __syncthreads();
  if (wave == 0) {
    const uint32_t c = lane & 31u, h = lane >> 5;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int s = acc[e] + red[0][e][lane] + red[1][e][lane] + red[2][e][lane];
      const uint32_t row = 8u * (e >> 2) + 4u * h + (e & 3u);
      if (row < a.M) a.acc_part[((size_t)ks * kSkinnyMaxRows + row) * (a.NB * 32u) + nb * 32u + c] = s;
    }
  }
}

// ---------------------------------------------------------------------------------------
struct SkinnyEpilogueArgs {
  const int32_t* acc_part;   // int32 [ksplit][32][NB*32], columns in packed order
  const float* z_part;       // f32 [z_chunks][32][kMaxRank]
  const float* sx;           // f32 [32]
  const float* sw;           // f32 [N]
  const uint16_t* lora_b;    // bf16 [n_adapters, r, N] or null
  const float* lora_scaling;
  const int32_t* idx;
  const uint16_t* residual;  // bf16 [M, N] or null
  uint16_t* out;             // bf16 [M, N]
  int32_t* aux_acc;          // int32 [M, N] or null
  uint32_t M, N, NB, ksplit, n_adapters, r, z_chunks;
};

__global__ __launch_bounds__(256) void skinny_epilogue_kernel(SkinnyEpilogueArgs a) {
  __shared__ float zs[4][kMaxRank];
  __shared__ float z[kMaxRank];
  const uint32_t m = blockIdx.y;
  const uint32_t tid = threadIdx.x;
  int ad = 0;
  float sgrp = 0.f;
  if (a.lora_b) {
    ad = a.idx ? a.idx[m] : 0;
    ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
    sgrp = a.lora_scaling[ad];
    // z[r] = sum over chunks, four interleaved partial sums combined in a fixed order
    const uint32_t r = tid & 63u, cg = tid >> 6;
    float s = 0.f;
#pragma unroll 4
    for (uint32_t ch = cg; ch < a.z_chunks; ch += 4u) s += a.z_part[((size_t)ch * kSkinnyMaxRows + m) * kMaxRank + r];
    zs[cg][r] = s;
  }
  __syncthreads();
  if (a.lora_b && tid < (uint32_t)kMaxRank) z[tid] = ((zs[0][tid] + zs[1][tid]) + zs[2][tid]) + zs[3][tid];
  __syncthreads();
  const uint32_t n = blockIdx.x * 256u + tid;
  if (n >= a.N) return;
  const uint32_t pc = orig_to_packed_col(n);
  int acc = 0;
#pragma unroll 8
  for (uint32_t ks = 0; ks < a.ksplit; ++ks) acc += a.acc_part[((size_t)ks * kSkinnyMaxRows + m) * (a.NB * 32u) + pc];
  if (a.aux_acc) a.aux_acc[(size_t)m * a.N + n] = acc;
  float y = ((float)acc * a.sx[m]) * a.sw[n];
  if (a.lora_b) {
    const uint16_t* Bp = a.lora_b + (size_t)ad * a.r * a.N + n;
    float low = 0.f;
    uint32_t r = 0;
    for (; r + 8u <= a.r; r += 8u) {
      float bv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[e] = bf16_bits_to_f32(Bp[(size_t)(r + e) * a.N]);
#pragma unroll
      for (int e = 0; e < 8; ++e) low = fmaf(z[r + e], bv[e], low);
    }
    for (; r < a.r; ++r) low = fmaf(z[r], bf16_bits_to_f32(Bp[(size_t)r * a.N]), low);
    const float l = low * sgrp;
    y = y + l;
  }
  if (a.residual) y = y + bf16_bits_to_f32(a.residual[(size_t)m * a.N + n]);
  a.out[(size_t)m * a.N + n] = (uint16_t)f32_to_bf16_bits(y);
}

}  // namespace w8a8
