// Skinny-M (decode) path, M <= 32 rows: the weight is streamed exactly once from HBM.
//   1. skinny_quant_kernel   one workgroup per row: (RMSNorm,) absmax, scale, int8 codes in
//                            MFMA operand order.
//                            LoRA-A units ride along: z_part[chunk][m][:] = x[m, chunk] @
//                            A[idx[m]][chunk, :] in float32 (a launch of their own when they
//                            need the normalized rows).
//   2. skinny_stream_kernel  every workgroup owns 16 weight columns for all of K: its eight waves
//                            stream the weight once from HBM straight into MFMA operands (no LDS:
//                            every byte is used once), are reduced through LDS, and the workgroup
//                            finishes its columns: (float(acc) * sx) * sw + s * (z @ B[idx[m]])
//                            + residual, one bf16 cast.
// Integer sums are exact and the float32 sums have a fixed order: results are bit-identical
// from run to run.  No atomics, no data crosses workgroups inside a launch.
#pragma once
#include "../../include/mi355_w8a8.h"
#include "w8a8_device.h"

namespace w8a8 {

constexpr int kSkinnyMaxRows = 32;
constexpr uint32_t kSkinnyMaxZChunks = 16;
constexpr uint32_t kSkinnyZChunkK = 1024;  // K elements per LoRA-A work unit (per row)

struct SkinnyLayout {
  uint64_t z_part, row_scaling, bsel, total;
  uint32_t pairs_per_wave, z_chunks, z_chunk_k;
};

inline SkinnyLayout skinny_layout(uint32_t m, uint32_t k, uint32_t n, uint32_t rank) {
  SkinnyLayout L{};
  const uint32_t n_pairs = k_padded(k) / 64u;
  L.pairs_per_wave = (n_pairs + 7u) / 8u;
  uint32_t zc = (k + kSkinnyZChunkK - 1u) / kSkinnyZChunkK;
  uint32_t zk = kSkinnyZChunkK;
  while (zc > kSkinnyMaxZChunks) { zk *= 2u; zc = (k + zk - 1u) / zk; }
  L.z_chunks = zc;
  L.z_chunk_k = zk;
  L.z_part = 0;
  L.row_scaling = (uint64_t)kSkinnyMaxZChunks * kSkinnyMaxRows * kMaxRank * 4u;
  L.bsel = L.row_scaling + 256u;
  // LoRA B regrouped for the stream kernel's finish step (skinny_regroup_b): [unit][row][rank half]
  // [column][16 ranks] bf16, for M <= 16 and rank <= 32
  const bool regroup = rank > 0 && rank <= 32u && m <= 16u;
  L.total = L.bsel + (regroup ? (uint64_t)(n_padded(n) / 16u) * m * 2u * 16u * 32u : 0u);
  return L;
}

inline uint64_t skinny_workspace_bytes(uint32_t m, uint32_t n, uint32_t rank) {
  return skinny_layout(m, 128u, n, rank).total;
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
  // need the normalized rows and run as a launch of their own
  const uint16_t* lora_a;  // bf16 [n_adapters, K, r] or null
  const int32_t* idx;      // adapter per row or null
  float* z_part;           // f32 [z_chunks][32][kMaxRank]
  uint32_t n_adapters, r, z_chunks, z_chunk_k, n_z_units;
  // LoRA-B regrouping items that share the launch (M <= 16, rank <= 32, N % 8 == 0), four per block
  const uint16_t* lora_b;  // bf16 [n_adapters, r, N] or null
  uint16_t* bsel;          // bf16 [N_pad/16 units][M][2][16][16]
  uint32_t N, n_groups;    // n_groups = N_pad / 128
  const float* lora_scaling;  // f32 [n_adapters] or null
  float* row_scaling;      // f32 [32]: lora_scaling[idx[m]], written here for the stream kernel
};

// The stream kernel's unit u = 8 G + 2 j + h owns the original columns 128 G + 4 (16 h + c) + j,
// c = 0..15, and its finish step needs, per row m and column c, the ranks of one parity:
//   bsel[u][m][p][c][t] = B[idx[m]][p + 2 t][128 G + 4 (16 h + c) + j],  t = 0..15
// so that a thread reads its 16 values as one 32-byte piece instead of 16 two-byte values that each
// cost a 128-byte line.  One item = (row m, column group G): its r x 128 tile of B goes through LDS.
__device__ inline void skinny_regroup_b(const SkinnyQuantArgs& a, uint32_t block, uint16_t (*tile)[32][128]) {
  const uint32_t team = threadIdx.x >> 8, t256 = threadIdx.x & 255u;
  const uint32_t item = block * 4u + team;
  const bool live = item < a.M * a.n_groups;
  const uint32_t m = live ? item / a.n_groups : 0u, G = live ? item % a.n_groups : 0u;
  int ad = a.idx ? a.idx[m] : 0;
  ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
  const uint16_t* Bsrc = a.lora_b + (size_t)ad * a.r * a.N + G * 128u;
#pragma unroll
  for (uint32_t u = 0; u < 2; ++u) {  // 32 ranks x 16 pieces of 8 columns
    const uint32_t piece = t256 + 256u * u, rr = piece >> 4, c8 = (piece & 15u) * 8u;
    v8us v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (live && rr < a.r && G * 128u + c8 < a.N) v = *reinterpret_cast<const v8us*>(Bsrc + (size_t)rr * a.N + c8);
    *reinterpret_cast<v8us*>(&tile[team][rr][c8]) = v;
  }
  __syncthreads();
  if (!live) return;
  const uint32_t u8 = t256 >> 5, par = (t256 >> 4) & 1u, c = t256 & 15u;
  const uint32_t col = 4u * (16u * (u8 & 1u) + c) + (u8 >> 1);
  v8us lo, hi;
#pragma unroll
  for (uint32_t t = 0; t < 8; ++t) {
    lo[t] = tile[team][par + 2u * t][col];
    hi[t] = tile[team][par + 2u * (t + 8u)][col];
  }
  uint16_t* dst = a.bsel + (((((size_t)G * 8u + u8) * a.M + m) * 2u + par) * 16u + c) * 16u;
  *reinterpret_cast<v8us*>(dst) = lo;
  *reinterpret_cast<v8us*>(dst + 8) = hi;
}

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
    if ((r & 7u) == 0) {
      // four rows of A per round, their loads issued together (same order of additions as a plain loop)
      for (uint32_t k = k_begin + kl; k < k_end; k += 4u * kpt) {
        v8us w[4];
        float xv[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
          const uint32_t ku = k + u * kpt;
          const bool in = ku < k_end;
          const v8us zero = {0, 0, 0, 0, 0, 0, 0, 0};
          w[u] = in ? *reinterpret_cast<const v8us*>(Ar + (size_t)ku * r + q * 8u) : zero;
          xv[u] = in ? bf16_bits_to_f32(xr[ku]) : 0.f;
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
          if (k + u * kpt < k_end) {
#pragma unroll
            for (int e = 0; e < 8; ++e) accz[e] = fmaf(xv[u], bf16_bits_to_f32(w[u][e]), accz[e]);
          }
        }
      }
    } else {
      for (uint32_t k = k_begin + kl; k < k_end; k += kpt) {
        const float xv = bf16_bits_to_f32(xr[k]);
        const uint16_t* src = Ar + (size_t)k * r + q * 8u;
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
  if (blockIdx.x >= a.M + a.n_z_units) {
    __shared__ __attribute__((aligned(16))) uint16_t tile[4][32][128];  // 32 KiB
    skinny_regroup_b(a, blockIdx.x - a.M - a.n_z_units, tile);
    return;
  }
  if (blockIdx.x >= a.M) {
    const uint32_t unit = blockIdx.x - a.M;
    skinny_lora_a_unit<1024>(a.x, a.lora_a, a.idx, a.z_part, unit, a.K, a.n_adapters, a.r, a.z_chunks,
                             a.z_chunk_k, zw);
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
    if (a.lora_scaling) {
      int ad = a.idx ? a.idx[m] : 0;
      ad = ad < 0 ? 0 : (ad >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad);
      a.row_scaling[m] = a.lora_scaling[ad];
    }
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
// LoRA-A units as a launch of their own (only when they need the normalized rows of the
// quantizer launch; otherwise they ride along with it).
struct SkinnyLoraAArgs {
  const uint16_t* xsrc; const uint16_t* lora_a; const int32_t* idx; float* z_part;
  uint32_t K, n_adapters, r, z_chunks, z_chunk_k;
};
__global__ __launch_bounds__(1024) void skinny_lora_a_kernel(SkinnyLoraAArgs a) {
  __shared__ float zw[16][64];
  skinny_lora_a_unit<1024>(a.xsrc, a.lora_a, a.idx, a.z_part, blockIdx.x, a.K, a.n_adapters, a.r, a.z_chunks,
                           a.z_chunk_k, zw);
}

// ---------------------------------------------------------------------------------------
constexpr uint32_t kSkinnyStreamWaves = 8;   // waves of a stream workgroup; they split K
constexpr uint32_t kSkinnyStreamThreads = kSkinnyStreamWaves * 64u;

struct SkinnyStreamArgs {
  const unsigned char* xq;   // packed codes of the single 32-row block
  const unsigned char* wp;   // packed weight
  const float* z_part;       // f32 [z_chunks][32][kMaxRank]
  const float* sx;           // f32 [32]
  const float* sw;           // f32 [N]
  const uint16_t* lora_b;    // bf16 [n_adapters, r, N] or null
  const uint16_t* bsel;      // B regrouped per unit (skinny_regroup_b) or null: then B is gathered directly
  const float* lora_scaling;
  const float* row_scaling;  // f32 [32]: lora_scaling[idx[m]] (from the quantizer launch)
  const int32_t* idx;        // adapter per row or null
  const uint16_t* residual;  // bf16 [M, N] or null
  uint16_t* out;             // bf16 [M, N]
  int32_t* aux_acc;          // int32 [M, N] or null
  uint32_t M, N, N_pad, K, KB, pairs_per_wave, n_adapters, r, z_chunks, n_groups;
};

// Every workgroup owns 16 packed weight columns for all of K and finishes them itself; nothing
// crosses workgroups.
//  * Its eight waves each stream a K range of the weight from HBM straight into
//    v_mfma_i32_16x16x64_i8 operands (a lane loads its 16 bytes from the 1 KiB fragment blocks:
//    column c of a block pair's four 16-wide k chunks) and are reduced through LDS.
//  * Finish: (float(acc) * sx) * sw + s * (z @ B) + residual, one bf16 cast.  z[m][r] is the
//    fixed-order sum of the LoRA-A partials; the rank sum runs in two fixed halves.
// Packed column pc of block nb is original column 128*(nb/4) + 4*pc + nb%4, so the eight units of
// a 128-column group read the same stretches of B; they are given workgroup ids that land on one
// XCD (ids are dealt round-robin to the XCDs) so that those stretches come from HBM once.
template <bool ROWS2>  // more than 16 rows: a second MFMA per step for rows 16..31
__global__ __launch_bounds__(kSkinnyStreamThreads) void skinny_stream_kernel(SkinnyStreamArgs a) {
  // 64-wide k steps a wave keeps in flight (1 KiB of weight each): 192 KiB per workgroup, one
  // workgroup per CU
  constexpr uint32_t kInFlight = ROWS2 ? 16 : 24;
  constexpr uint32_t kRankSplit = ROWS2 ? 1 : 2;  // threads per output in the finish step
  __shared__ __attribute__((aligned(16))) int red[kSkinnyStreamWaves][2][4][64];  // 16 KiB
  __shared__ float zl[kSkinnyMaxRows][kMaxRank];                                 // 8 KiB
  __shared__ float low_odd[256];
  // one-round form: the finish step's LoRA operands, staged by direct-to-LDS loads behind the weight stream
  __shared__ __attribute__((aligned(1024))) float zst[ROWS2 ? 1 : kSkinnyMaxZChunks][16][32];  // z partials [chunk][row][rank], 32 KiB
  __shared__ __attribute__((aligned(1024))) uint16_t bst[ROWS2 ? 8 : 16 * 2 * 16 * 16];         // the unit's regrouped B, 16 KiB
  __shared__ __attribute__((aligned(1024))) uint32_t fst[4][256];  // per output thread: sx, sw, the row's LoRA scaling, the residual's dword
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t slot = blockIdx.x >> 3;
  const uint32_t grp = (slot >> 3) * 8u + (blockIdx.x & 7u);
  if (grp >= a.n_groups) return;
  const uint32_t nb = grp * 4u + ((slot & 7u) >> 1), chalf = slot & 1u;
  const uint32_t c16 = lane & 15u, q = lane >> 4;        // MFMA operand: column / row c16, k chunk q
  const uint32_t pc = 16u * chalf + c16;                 // packed column inside block nb
  // byte offsets inside a pair of 1 KiB blocks: chunk q sits in block q/2, k half q%2
  const uint32_t w_lane_off = (q >> 1) * kBlockBytes + (pc + 32u * (q & 1u)) * 16u;
  const uint32_t x_lane_off = (q >> 1) * kBlockBytes + (c16 + 32u * (q & 1u)) * 16u;
  const unsigned char* wsrc = a.wp + (size_t)nb * a.KB * kBlockBytes + w_lane_off;
  const unsigned char* xsrc = a.xq + x_lane_off;
  const uint32_t n_pairs = a.KB >> 1;
  uint32_t p0 = wave * a.pairs_per_wave, p1 = p0 + a.pairs_per_wave;
  if (p0 > n_pairs) p0 = n_pairs;
  if (p1 > n_pairs) p1 = n_pairs;

  // ---- finish step mapping: thread -> output (row frow, packed column pc) and a rank share
  const uint32_t fe = (tid >> 6) & 3u;
  const uint32_t frow = (ROWS2 ? 16u * (tid >> 8) : 0u) + 4u * q + fe;
  const uint32_t rsel = ROWS2 ? 0u : (tid >> 8);  // ranks rsel, rsel + kRankSplit, ...
  const uint32_t fn = 128u * (nb >> 2) + 4u * pc + (nb & 3u);
  const bool fvalid = frow < a.M && fn < a.N;
  const bool lora = a.lora_b != nullptr;
  // Lanes without an output read element 0 instead of selecting on the loaded value.
  const uint32_t srow = fvalid ? frow : 0u, scol = fvalid ? fn : 0u;
  // z[m][r] share of this thread: value index tid (and tid + 512, ...) of the M x rpad values
  const uint32_t rpad = (a.r + 7u) & ~7u;
  const uint32_t n_zval = lora ? a.M * rpad : 0u;
  // With B regrouped per unit the low-rank term needs three independent, coalesced requests per
  // thread: its 16 ranks of B, its z partials, its row's scaling.
  const bool early = !ROWS2 && lora && a.bsel != nullptr && n_zval <= kSkinnyStreamThreads;  // workgroup-uniform
  float low = 0.f, f_s = 0.f, f_sx, f_sw;
  uint16_t res_raw = 0;
  v4i acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};

  // ---- One round: every wave's share of K is exactly what it keeps in flight (K = 512 * kInFlight: the
  // Qwen3-8B down projection), and the low-rank term, if any, has its regrouped B.
  //  * What the finish step works with (the unit's regrouped B, the z partials of all rows, every output's
  //    scales and residual) takes no registers -- the operands of the MFMAs take all there are, and a
  //    value loaded beside them is spilled behind a wait for the whole stream -- the waves copy it into
  //    the LDS with direct-to-LDS loads, the first loads they issue.
  //  * Then the code and the weight loads go out, nothing waited for, spilled or converted in front of
  //    them.
  //  * While the weight is on its way the low-rank term is formed from the LDS (a wave's loads return in
  //    order: a wait that leaves only the code and weight loads outstanding has the staged pieces).
  //  * The MFMAs run as their operands arrive, and what is left behind them is the sum over the waves and
  //    one line of float32 arithmetic per output.
  const bool one_round = !ROWS2 && n_pairs == kSkinnyStreamWaves * kInFlight && (!lora || early);  // workgroup-uniform
  if (one_round) {
    // the staged operands first: a handful of instructions, and their data is then in the LDS long before
    // the weight is in the registers
    const uint32_t res_elem = srow * a.N + scol;  // (M * N is below 2^32)
    if (lora) {  // kernel-uniform
      const uint32_t unit = grp * 8u + (slot & 7u);
      const unsigned char* bsrc = reinterpret_cast<const unsigned char*>(a.bsel) + (size_t)unit * a.M * 1024u;  // M KiB, contiguous
      const uint32_t bst_addr = (uint32_t)(uintptr_t)(lptr_t)bst, zst_addr = (uint32_t)(uintptr_t)(lptr_t)zst;
      for (uint32_t i = wave; i < a.M; i += kSkinnyStreamWaves) lds_load_1k(bsrc, i * 1024u + lane * 16u, bst_addr + i * 1024u);
      // z partials: per chunk the first 32 ranks of rows 0..15, two pieces of eight rows x 128 bytes
      for (uint32_t i = wave; i < 2u * a.z_chunks; i += kSkinnyStreamWaves) {
        const uint32_t ch = i >> 1, h = i & 1u;
        const uint32_t voff = ((ch * (uint32_t)kSkinnyMaxRows + 8u * h + (lane >> 3)) * (uint32_t)kMaxRank) * 4u + (lane & 7u) * 16u;
        lds_load_1k(reinterpret_cast<const unsigned char*>(a.z_part), voff, zst_addr + i * 1024u);
      }
      // the chunk slots no unit has written count as zeros, so that the sum below needs no conditions
      for (uint32_t i = a.z_chunks * 128u + tid; i < kSkinnyMaxZChunks * 128u; i += kSkinnyStreamThreads)
        reinterpret_cast<float4*>(&zst[0][0][0])[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (wave < 4u) {  // the output threads: thread tid finds its four values at fst[.][tid]
      const uint32_t fst_addr = (uint32_t)(uintptr_t)(lptr_t)fst + wave * 256u;
      lds_gather_dword(a.sx, srow * 4u, fst_addr);
      lds_gather_dword(a.sw, scol * 4u, fst_addr + 1024u);
      if (lora) lds_gather_dword(a.row_scaling, srow * 4u, fst_addr + 2048u);
      if (a.residual) lds_gather_dword(a.residual, (res_elem * 2u) & ~3u, fst_addr + 3072u);
    }
    v4i wf[kInFlight], xf[kInFlight];
    const unsigned char* wb = wsrc + (size_t)p0 * 2u * kBlockBytes;
    const unsigned char* xb = xsrc + (size_t)p0 * 2u * kBlockBytes;
    // (the codes first: they come from the L2 and are in the registers long before the weight, whose
    // requests the memory takes at its own pace)
#pragma unroll
    for (uint32_t t = 0; t < kInFlight; ++t) xf[t] = *reinterpret_cast<const v4i*>(xb + t * 2u * kBlockBytes);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (uint32_t t = 0; t < kInFlight; ++t)
      wf[t] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wb + t * 2u * kBlockBytes));
    __builtin_amdgcn_sched_barrier(0);
    // ---- the low-rank term, while the weight is on its way: the staged operands are the wave's oldest
    // loads, so a wait that leaves the code and weight loads outstanding has them
    if (lora) {
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * kInFlight) : "memory");
      __syncthreads();  // ... and the other waves' pieces
      {  // z[m][r] for 16 rows x 32 ranks, one per thread: four interleaved partial sums, combined in a fixed order
        const uint32_t zr = tid >> 5, zc = tid & 31u;
        float zv[kSkinnyMaxZChunks];
#pragma unroll
        for (uint32_t ch = 0; ch < kSkinnyMaxZChunks; ++ch) zv[ch] = zst[ch][zr][zc];
        float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t ch = 0; ch < kSkinnyMaxZChunks; ++ch) s4[ch & 3u] += zv[ch];
        zl[zr][zc] = ((s4[0] + s4[1]) + s4[2]) + s4[3];
      }
      __syncthreads();
      if (wave < 4u) {  // the output threads
        // the even and the odd ranks as two chains, added at the end: the order of the two-thread form.
        // (Ranks beyond the rank are zeros in z and in the regrouped B alike: they add nothing.)
        float zrow[32];
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) {
          const float4 z4 = *reinterpret_cast<const float4*>(&zl[srow][4u * i]);
          zrow[4 * i] = z4.x; zrow[4 * i + 1] = z4.y; zrow[4 * i + 2] = z4.z; zrow[4 * i + 3] = z4.w;
        }
        float lo2[2] = {0.f, 0.f};
#pragma unroll
        for (uint32_t par = 0; par < 2; ++par) {
          const uint16_t* bl = bst + ((srow * 2u + par) * 16u + c16) * 16u;
          const v8us blo = *reinterpret_cast<const v8us*>(bl), bhi = *reinterpret_cast<const v8us*>(bl + 8);
#pragma unroll
          for (uint32_t t = 0; t < 16; ++t) {
            const uint16_t bv = t < 8u ? blo[t & 7u] : bhi[t & 7u];
            lo2[par] = fmaf(zrow[par + 2u * t], bf16_bits_to_f32(bv), lo2[par]);
          }
        }
        low = lo2[0] + lo2[1];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // four accumulators take turns, so that no MFMA waits for the one before it (integer sums: any order)
    v4i part[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
    for (uint32_t t = 0; t < kInFlight; ++t) part[t & 3u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[t], wf[t], part[t & 3u], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][0][e][lane] = (part[0][e] + part[1][e]) + (part[2][e] + part[3][e]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (without LoRA nothing has waited for the staged scales yet)
    __syncthreads();  // the accumulators of every wave
    if (wave >= 4u) return;  // one thread per output from here on
    f_sx = __uint_as_float(fst[0][tid]);
    f_sw = __uint_as_float(fst[1][tid]);
    if (a.residual) res_raw = (uint16_t)((res_elem & 1u) ? fst[3][tid] >> 16 : fst[3][tid] & 0xffffu);
    if (lora) f_s = __uint_as_float(fst[2][tid]);
  } else {
  f_sx = a.sx[srow];
  f_sw = a.sw[scol];
  int ad_raw = 0;
  if (lora && a.idx) ad_raw = a.idx[srow];
  // The low-rank term's requests go out ahead of the weight loads: a wave's loads return in order, so they
  // are back while the weight is still streaming, and the term is computed under the stream.
  v8us blo = {0, 0, 0, 0, 0, 0, 0, 0}, bhi = {0, 0, 0, 0, 0, 0, 0, 0};
  float zv[kSkinnyMaxZChunks];
  if (early) {
    if (a.residual) res_raw = a.residual[(size_t)srow * a.N + scol];
    f_s = a.row_scaling[srow];
    const uint32_t unit = grp * 8u + (slot & 7u);
    const uint16_t* bs = a.bsel + (((((size_t)unit * a.M + srow) * 2u + rsel) * 16u + c16) * 16u);
    blo = *reinterpret_cast<const v8us*>(bs);
    bhi = *reinterpret_cast<const v8us*>(bs + 8);
    const uint32_t zi = tid < n_zval ? tid : 0u;
    const float* zp = a.z_part + (size_t)(zi / rpad) * kMaxRank + zi % rpad;
#pragma unroll
    for (uint32_t ch = 0; ch < kSkinnyMaxZChunks; ++ch)
      zv[ch] = ch < a.z_chunks ? zp[(size_t)ch * kSkinnyMaxRows * kMaxRank] : 0.f;
  }
  __builtin_amdgcn_sched_barrier(0);  // the weight loads below are issued after the requests above
  uint32_t base = p0;
  do {
    v4i wf[kInFlight], xf[kInFlight], xg[ROWS2 ? kInFlight : 1];
#pragma unroll
    for (uint32_t t = 0; t < kInFlight; ++t) {
      const uint32_t pr = base + t < p1 ? base + t : (p1 ? p1 - 1u : 0u);  // clamped: repeats are skipped below
      wf[t] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wsrc + (size_t)pr * 2u * kBlockBytes));
    }
#pragma unroll
    for (uint32_t t = 0; t < kInFlight; ++t) {
      const uint32_t pr = base + t < p1 ? base + t : (p1 ? p1 - 1u : 0u);
      xf[t] = *reinterpret_cast<const v4i*>(xsrc + (size_t)pr * 2u * kBlockBytes);
      if constexpr (ROWS2) xg[t] = *reinterpret_cast<const v4i*>(xsrc + (size_t)pr * 2u * kBlockBytes + 256u);
    }
    if (early && base == p0) {  // workgroup-uniform: the low-rank term, under the first round's loads
      __builtin_amdgcn_sched_barrier(0);
      if (tid < n_zval) {  // z[m][r]: four interleaved partial sums, combined in a fixed order
        float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t ch = 0; ch < kSkinnyMaxZChunks; ++ch) s4[ch & 3u] += zv[ch];
        zl[tid / rpad][tid % rpad] = ((s4[0] + s4[1]) + s4[2]) + s4[3];
      }
      __syncthreads();
#pragma unroll
      for (uint32_t t = 0; t < 16; ++t) {
        const uint32_t r = rsel + kRankSplit * t;
        const uint16_t bv = t < 8u ? blo[t & 7u] : bhi[t & 7u];
        if (r < a.r) low = fmaf(zl[srow][r], bf16_bits_to_f32(bv), low);
      }
      if (rsel == 1u) low_odd[tid & 255u] = low;  // the two rank halves of an output, added in a fixed order
      __syncthreads();
      if (rsel == 0u) low = low + low_odd[tid];
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (uint32_t t = 0; t < kInFlight; ++t) {
      if (base + t < p1) {  // wave-uniform
        acc0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[t], wf[t], acc0, 0, 0, 0);
        if constexpr (ROWS2) acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xg[t], wf[t], acc1, 0, 0, 0);
      }
    }
    base += kInFlight;
  } while (base < p1);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    red[wave][0][e][lane] = acc0[e];
    red[wave][1][e][lane] = acc1[e];
  }
  if (!early) {
    // Without the regrouped B the term's loads start only now: issued while the weight stream is in
    // flight they would be served after it anyway, and here they cost one trip to an idle memory.
    if (a.residual) res_raw = a.residual[(size_t)srow * a.N + scol];
    const int ad = ad_raw < 0 ? 0 : (ad_raw >= (int)a.n_adapters ? (int)a.n_adapters - 1 : ad_raw);
    f_s = (fvalid && lora) ? a.lora_scaling[ad] : 0.f;
    // Every B value of the thread (ranks rsel, rsel + kRankSplit, ... below 64) is requested before the
    // first is used: one trip to memory instead of one per value.
    // The loads are unconditional (a load under a lane condition gets a branch and a wait of its own):
    // lanes without an output read column 0, ranks beyond the rank read the last one; both are skipped
    // when the values are used.
    constexpr uint32_t kBValues = (uint32_t)kMaxRank / kRankSplit;
    uint32_t bq[kBValues];
    if (lora) {  // kernel-uniform
      const uint16_t* Bs = a.lora_b + (size_t)ad * a.r * a.N + scol;
#pragma unroll
      for (uint32_t t = 0; t < kBValues; ++t) {
        uint32_t r = rsel + kRankSplit * t;
        r = r < a.r ? r : a.r - 1u;
        bq[t] = (uint32_t)Bs[(size_t)r * a.N];
      }
    }
    for (uint32_t zi = tid; zi < n_zval; zi += kSkinnyStreamThreads) {
      const float* zp = a.z_part + (size_t)(zi / rpad) * kMaxRank + zi % rpad;
      float zw4[kSkinnyMaxZChunks];
#pragma unroll
      for (uint32_t ch = 0; ch < kSkinnyMaxZChunks; ++ch)
        zw4[ch] = ch < a.z_chunks ? zp[(size_t)ch * kSkinnyMaxRows * kMaxRank] : 0.f;
      float s4[4] = {0.f, 0.f, 0.f, 0.f};  // four interleaved partial sums, combined in a fixed order
#pragma unroll
      for (uint32_t ch = 0; ch < kSkinnyMaxZChunks; ++ch) s4[ch & 3u] += zw4[ch];
      zl[zi / rpad][zi % rpad] = ((s4[0] + s4[1]) + s4[2]) + s4[3];
    }
    __syncthreads();
    if (fvalid && lora) {
#pragma unroll
      for (uint32_t t = 0; t < kBValues; ++t) {
        const uint32_t r = rsel + kRankSplit * t;
        if (r < a.r) low = fmaf(zl[frow][r], bf16_bits_to_f32(bq[t]), low);
      }
    }
    if (!ROWS2) {
      if (rsel == 1u) low_odd[tid & 255u] = low;
      __syncthreads();
      if (rsel == 0u) low = low + low_odd[tid];
    }
  } else {
    __syncthreads();  // the accumulators in `red`
  }
  }
  if (!ROWS2 && rsel == 1u) return;  // (only the multi-round form gets here with rsel == 1)
  if (!fvalid) return;
  int sum = 0;
#pragma unroll
  for (uint32_t w = 0; w < kSkinnyStreamWaves; ++w) sum += red[w][ROWS2 ? (tid >> 8) : 0u][fe][lane];
  float y = ((float)sum * f_sx) * f_sw;
  if (lora) {
    const float l = low * f_s;
    y = y + l;
  }
  const size_t o = (size_t)frow * a.N + fn;
  if (a.residual) y = y + bf16_bits_to_f32(res_raw);
  a.out[o] = (uint16_t)f32_to_bf16_bits(y);
  if (a.aux_acc) a.aux_acc[o] = sum;
}

}  // namespace w8a8
