// Prologue kernels: weight (un)packing, adapter routing, per-token quantization with the
// optional fused RMSNorm, and the LoRA-A projection z = n @ A[adapter].
#pragma once
#include "w8a8_device.h"

namespace w8a8 {

// ---------------------------------------------------------------------------------------
// Weight pack / unpack (one time per weight)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pack_weight_kernel(const int8_t* __restrict__ codes,
                                                          unsigned char* __restrict__ packed, uint32_t K,
                                                          uint32_t N, uint32_t KB, uint64_t n_chunks) {
  uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte chunk per thread
  if (idx >= n_chunks) return;
  uint32_t lane = idx & 63u;
  uint64_t blk = idx >> 6;
  uint32_t kb = (uint32_t)(blk % KB);
  uint32_t nb = (uint32_t)(blk / KB);
  uint32_t c = nb * 32u + (lane & 31u);
  uint32_t n = packed_to_orig_col(c);
  uint32_t k0 = kb * 32u + 16u * (lane >> 5);
  uint32_t w[4] = {0, 0, 0, 0};
  if (n < N) {
#pragma unroll
    for (int b = 0; b < 16; ++b) {
      uint32_t k = k0 + b;
      uint32_t v = (k < K) ? (uint32_t)(uint8_t)codes[(size_t)k * N + n] : 0u;
      w[b >> 2] |= v << (8 * (b & 3));
    }
  }
  uint4 o = make_uint4(w[0], w[1], w[2], w[3]);
  *reinterpret_cast<uint4*>(packed + idx * 16) = o;
}

__global__ __launch_bounds__(256) void unpack_weight_kernel(const unsigned char* __restrict__ packed,
                                                            int8_t* __restrict__ codes, uint32_t K, uint32_t N,
                                                            uint32_t KB) {
  uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (uint64_t)K * N) return;
  uint32_t k = (uint32_t)(idx / N), n = (uint32_t)(idx % N);
  codes[idx] = (int8_t)packed[packed_offset(orig_to_packed_col(n), k, KB)];
}

// ---------------------------------------------------------------------------------------
// Adapter routing: rows are grouped by adapter with no padding between groups (the
// counterpart of prepare_routing, skyrl/tx/layers/util.py:66-87).
//   src_row[p]    = original row of grouped slot p (p < M), -1 for the slots beyond M
//   dst_pos[m]    = grouped slot of original row m
//   slot_group[p] = adapter of grouped slot p
//   blk_range[b]  = first adapter | last adapter << 16 of the 32-row block b
//   group_off[a]  = first grouped slot of adapter a (optional; entry n_groups = M)
// Out-of-range adapter indices are clamped into range (XLA gather semantics).
// One workgroup.  The order of rows inside a group does not influence any forward result; the
// backward asks for the stable order because it sums over a group's rows.
// ---------------------------------------------------------------------------------------
// With group_pad = 32 every group starts on a 32-slot boundary (see route_rows_inline): the slots between
// a group's last row and the next group's first stay empty.
__device__ inline void route_rows_block(const int32_t* __restrict__ idx, uint32_t M, uint32_t n_groups,
                                        uint32_t slots, int32_t* __restrict__ src_row,
                                        int32_t* __restrict__ dst_pos, int32_t* __restrict__ slot_group,
                                        int32_t* __restrict__ blk_range, int32_t* __restrict__ group_off = nullptr,
                                        bool stable = false, uint32_t group_pad = 1u) {
  __shared__ int cnt[kMaxAdapters];
  __shared__ int start[kMaxAdapters + 1];
  __shared__ int cursor[kMaxAdapters];
  const uint32_t tid = threadIdx.x;
  if (tid < kMaxAdapters) { cnt[tid] = 0; cursor[tid] = 0; }
  __syncthreads();
  for (uint32_t i = tid; i < M; i += 1024) {
    int a = idx[i];
    a = a < 0 ? 0 : (a >= (int)n_groups ? (int)n_groups - 1 : a);
    atomicAdd(&cnt[a], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int pos = 0;
    for (uint32_t a = 0; a < n_groups; ++a) {
      start[a] = pos;
      pos += (int)round_up((uint32_t)cnt[a], group_pad);
    }
    start[n_groups] = pos;
  }
  __syncthreads();
  const uint32_t E = (uint32_t)start[n_groups];  // first slot behind the last group (M when the groups are packed)
  if (group_pad > 1u)
    for (uint32_t p = tid; p < E && p < slots; p += 1024) src_row[p] = -1;  // the empty slots between groups
  __syncthreads();
  if (group_off && tid <= n_groups) group_off[tid] = start[tid];  // first slot of every group, then M
  if (stable) {
    // rows keep their order inside a group (reductions over a group's rows then have a fixed order):
    // rank = rows of the same group before this one, counted per wave with ballots, per 1024-row
    // chunk with the waves' counts, and across chunks with the running count in cursor[]
    __shared__ int wave_cnt[16][kMaxAdapters];
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    for (uint32_t base = 0; base < M; base += 1024) {
      const uint32_t i = base + tid;
      int a = -1;
      if (i < M) {
        a = idx[i];
        a = a < 0 ? 0 : (a >= (int)n_groups ? (int)n_groups - 1 : a);
      }
      int rank = 0;
      for (uint32_t g = 0; g < n_groups; ++g) {
        const unsigned long long mask = __builtin_amdgcn_ballot_w64(a == (int)g);
        if (a == (int)g) rank = __builtin_popcountll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_cnt[wave][g] = __builtin_popcountll(mask);
      }
      __syncthreads();
      if (a >= 0) {
        int off = cursor[a];
        for (uint32_t w = 0; w < wave; ++w) off += wave_cnt[w][a];
        const int p = start[a] + off + rank;
        src_row[p] = (int)i;
        dst_pos[i] = p;
      }
      __syncthreads();
      if (tid < n_groups) {
        int t = 0;
        for (uint32_t w = 0; w < 16; ++w) t += wave_cnt[w][tid];
        cursor[tid] += t;
      }
      __syncthreads();
    }
  } else {
    for (uint32_t i = tid; i < M; i += 1024) {
      int a = idx[i];
      a = a < 0 ? 0 : (a >= (int)n_groups ? (int)n_groups - 1 : a);
      const int p = start[a] + atomicAdd(&cursor[a], 1);
      src_row[p] = (int)i;
      dst_pos[i] = p;
    }
  }
  // group of a slot = the group whose [start, next start) range holds it
  for (uint32_t p = tid; p < slots; p += 1024) {
    int g = 0;
    if (p < E) {
      for (uint32_t a = 0; a < n_groups; ++a)
        if ((int)p >= start[a] && (int)p < start[a + 1]) g = (int)a;
    } else {
      src_row[p] = -1;
      for (uint32_t a = 0; a < n_groups; ++a)
        if (cnt[a] > 0) g = (int)a;  // padding slots follow the last non-empty group
    }
    slot_group[p] = g;
  }
  for (uint32_t b = tid; b < slots / 32u; b += 1024) {
    const int p0 = (int)b * 32, p1 = (p0 + 31 < (int)E) ? p0 + 31 : (int)E - 1;
    int g0 = 0, g1 = 0;
    for (uint32_t a = 0; a < n_groups; ++a) {
      if (p0 >= start[a] && p0 < start[a + 1]) g0 = (int)a;
      if (p1 >= start[a] && p1 < start[a + 1]) g1 = (int)a;
    }
    if (p0 >= (int)E) { g0 = 0; g1 = 0; }
    blk_range[b] = g0 | (g1 << 16);
  }
}

// ---------------------------------------------------------------------------------------
// Tables for rows that arrive already grouped (ragged groups of an expert layer,
// skyrl/tx/layers/util.py:8-59): group g owns group_sizes[g] consecutive rows and is padded
// to a multiple of `pad` (64 or 128) grouped slots so that a GEMM tile never mixes two weights.
//   src_row[p]   = original row of slot p, -1 for padding
//   dst_pos[m]   = slot of row m, -1 for rows beyond sum(group_sizes) (their output is zero)
//   blk_range[b] = g | g << 16 for the 32-row blocks in use, -1 beyond
// ---------------------------------------------------------------------------------------
constexpr int kMaxGroups = 1024;
// Exclusive prefix sums of one value per thread over a workgroup of 1024 threads, every partial sum capped
// at `limit` (a capped sum of non-negative terms does not depend on the order they are added in).  Returns
// the thread's prefix; *total receives the sum of all.
__device__ inline uint32_t block_prefix_capped(uint32_t v, uint32_t limit, uint32_t* total) {
  __shared__ uint32_t wave_sum[17];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  auto add = [&](uint32_t x, uint32_t y) { const uint64_t t = (uint64_t)x + y; return t > limit ? limit : (uint32_t)t; };
  uint32_t incl = v > limit ? limit : v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
    if ((int)lane >= off) incl = add(incl, up);
  }
  __syncthreads();  // (the table may still be read from a call before)
  if (lane == 63u) wave_sum[wave] = incl;
  __syncthreads();
  if (tid == 0) {
    uint32_t run = 0;
    for (int w = 0; w < 16; ++w) {
      const uint32_t t = wave_sum[w];
      wave_sum[w] = run;
      run = add(run, t);
    }
    wave_sum[16] = run;
  }
  __syncthreads();
  *total = wave_sum[16];
  // exclusive: the waves before, then the lanes before (the capped sum up to the lane before)
  const uint32_t before = (uint32_t)__shfl_up((int)incl, 1, 64);
  return add(wave_sum[wave], lane ? before : 0u);
}

// Part `part` of `n_parts` workgroups of 1024 threads: every part forms the prefix sums for itself (at most
// 1024 groups, one per thread) and fills its share of the tables, slot by slot.  Group g keeps
// min(size, rows left) rows, as a sequential pass over the sizes would give it.  Rows beyond
// sum(group_sizes) get no slot; their output rows (zero_out, bf16 [M, zero_cols], optional) are cleared here.
__device__ inline void route_groups_block(const int32_t* __restrict__ group_sizes, uint32_t M, uint32_t n_groups,
                                          uint32_t slots, int32_t* __restrict__ src_row,
                                          int32_t* __restrict__ dst_pos, int32_t* __restrict__ blk_range,
                                          uint32_t pad, uint16_t* __restrict__ zero_out, uint32_t zero_cols,
                                          uint32_t part, uint32_t n_parts) {
  __shared__ uint32_t row_start[kMaxGroups + 1];
  __shared__ uint32_t slot_start[kMaxGroups + 1];
  const uint32_t tid = threadIdx.x;
  int32_t sz = tid < n_groups ? group_sizes[tid] : 0;
  if (sz < 0) sz = 0;
  uint32_t rows_total, slots_total;
  const uint32_t r0 = block_prefix_capped((uint32_t)sz, M, &rows_total);
  // the group's rows after the cap: up to the next group's start
  const uint32_t r1 = (uint64_t)r0 + (uint32_t)sz > M ? M : r0 + (uint32_t)sz;
  const uint32_t padded = (r1 - r0 + pad - 1u) & ~(pad - 1u);
  const uint32_t p0 = block_prefix_capped(padded, 0xffffffffu, &slots_total);
  if (tid < n_groups) { row_start[tid] = r0; slot_start[tid] = p0; }
  if (tid == 0) { row_start[n_groups] = rows_total; slot_start[n_groups] = slots_total; }
  __syncthreads();
  const uint32_t stride = n_parts * 1024u;
  for (uint32_t p = part * 1024u + tid; p < slots; p += stride) {
    int src = -1, range = -1;
    if (p < slots_total) {
      // the last group whose first slot is not behind p (empty groups share their successor's first slot)
      uint32_t lo = 0, hi = n_groups;  // slot_start[lo] <= p < slot_start[hi]
      while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if (slot_start[mid] <= p) lo = mid; else hi = mid;
      }
      const uint32_t i = p - slot_start[lo];
      if (i < row_start[lo + 1u] - row_start[lo]) {
        src = (int)(row_start[lo] + i);
        dst_pos[src] = (int)p;
      }
      range = (int)(lo | (lo << 16));
    }
    src_row[p] = src;
    if ((p & 31u) == 0) blk_range[p >> 5] = range;
  }
  for (uint32_t i = rows_total + part * 1024u + tid; i < M; i += stride) dst_pos[i] = -1;
  if (zero_out) {
    const size_t begin = (size_t)rows_total * zero_cols, end = (size_t)M * zero_cols;
    for (size_t i = begin + part * 1024u + tid; i < end; i += stride) zero_out[i] = 0;
  }
}

// ---------------------------------------------------------------------------------------
// Per-token dynamic int8 quantization (skyrl/tx/kernels/quantized_lora.py:199-212 with one
// group per row), optionally preceded by RMSNorm
// (skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu.py:299-303).  One wave per row; the
// row lives in registers (NCH chunks of 8 bf16 per lane).  Bit-exact rules:
//   scale = amax > 0 ? amax / 127 : 1         IEEE float32 division
//   code  = clamp(rint(v / scale), -127, 127) IEEE division, round half to even
//   RMSNorm: mean = float(sum_f64(x*x) / K), inv = 1 / sqrt(mean + eps) (IEEE), and
//            n = bf16((x * inv) * gamma) with two separate float32 multiplications.
// ---------------------------------------------------------------------------------------
struct QuantArgs {
  const uint16_t* x;       // bf16 [M, K]
  const float* gamma;      // f32 [K] or null
  float eps;
  uint32_t M, K, K_pad, KB;
  const int32_t* dst_pos;  // grouped slot per row or null (identity)
  unsigned char* xq_packed;// packed codes or null
  float* sx_slots;         // f32 per grouped slot or null
  int8_t* codes_rm;        // row-major codes [M, K] or null
  float* scales_rm;        // f32 [M] or null
  uint16_t* xn;            // bf16 [M, K] normalized rows or null
  uint16_t* xn_aux;        // second copy for the caller or null
  uint16_t* zero_out;      // bf16 [M, zero_cols]: rows without a slot (dst_pos < 0) are zero-filled
  uint32_t zero_cols;
  uint32_t* tile_ctr;      // 256 words cleared for the GEMM launches' tile counters, or null
  // Optional gather on the way in: row m is read from x[row_map[m] / row_div] (the sorted (token,
  // choice) pairs of an expert layer read their token's row; x then has the tokens' row count,
  // row_limit, to which the source row is clamped)
  const int32_t* row_map;
  uint32_t row_div, row_limit;
};

// source row of a gathered read: map value / divisor, clamped into [0, limit)
__device__ inline uint32_t mapped_row(int32_t value, uint32_t div, uint32_t limit) {
  const uint32_t r = value < 0 ? 0u : (uint32_t)value / div;
  return r < limit ? r : limit - 1u;
}

template <int NCH, bool RMS>
__global__ __launch_bounds__(256) void quant_rows_kernel(QuantArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t m = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (a.tile_ctr && blockIdx.x == 0) a.tile_ctr[threadIdx.x] = 0u;
  if (m >= a.M) return;
  const uint32_t xrow = a.row_map ? mapped_row(a.row_map[m], a.row_div, a.row_limit) : m;
  const uint16_t* xr = a.x + (size_t)xrow * a.K;
  float v[NCH][8];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    uint32_t k0 = (j * 64u + lane) * 8u;
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (k0 < a.K) raw = *reinterpret_cast<const uint4*>(xr + k0);
    uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[j][2 * e] = __uint_as_float(w[e] << 16);
      v[j][2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
    }
  }
  if (RMS) {
    double ss = 0.0;
#pragma unroll
    for (int j = 0; j < NCH; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += (double)v[j][e] * (double)v[j][e];
    ss = wave_sum(ss);
    float var = (float)(ss / (double)a.K);
    float inv = 1.0f / sqrtf(var + a.eps);
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      uint32_t k0 = (j * 64u + lane) * 8u;
      if (k0 < a.K) {
        float4 g0 = *reinterpret_cast<const float4*>(a.gamma + k0);
        float4 g1 = *reinterpret_cast<const float4*>(a.gamma + k0 + 4);
        float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        uint32_t packed[4];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float t = v[j][e] * inv;
          t = t * g[e];
          uint32_t b = f32_to_bf16_bits(t);
          v[j][e] = __uint_as_float(b << 16);
          if (e & 1) packed[e >> 1] |= b << 16; else packed[e >> 1] = b;
        }
        uint4 o = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        if (a.xn) *reinterpret_cast<uint4*>(a.xn + (size_t)m * a.K + k0) = o;
        if (a.xn_aux) *reinterpret_cast<uint4*>(a.xn_aux + (size_t)m * a.K + k0) = o;
      }
    }
  }
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < NCH; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[j][e]));
  amax = wave_max(amax);
  const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
  const int p = a.dst_pos ? a.dst_pos[m] : (int)m;
  if (p < 0 && a.zero_out) {
    for (uint32_t cidx = lane; cidx < a.zero_cols; cidx += 64u) a.zero_out[(size_t)m * a.zero_cols + cidx] = 0;
  }
  if (lane == 0) {
    if (a.sx_slots && p >= 0) a.sx_slots[p] = scale;
    if (a.scales_rm) a.scales_rm[m] = scale;
  }
  // codes = rint(v / scale) with the correctly rounded quotient, as in quant_lora_kernel: v * (1 / scale)
  // with the hardware reciprocal rounds to the same integer unless the product lies within 1e-4 of a
  // tie; those cases (and scales outside the reciprocal's safe range) are redone with the division.
  const float rscale = __builtin_amdgcn_rcpf(scale);
  const bool scale_safe = scale > 1e-30f && scale < 1e30f;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    uint32_t c = j * 64u + lane;
    uint32_t k0 = c * 8u;
    if (k0 >= a.K_pad) continue;
    uint32_t lo = 0, hi = 0;
    if (k0 < a.K) {
      float q[8];
      float off_integer = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float t = v[j][e] * rscale;
        q[e] = rintf(t);
        off_integer = fmaxf(off_integer, fabsf(t - q[e]));
      }
      if (!scale_safe || off_integer > 0.4999f) {
#pragma unroll
        for (int e = 0; e < 8; ++e) q[e] = rintf(v[j][e] / scale);
      }
      // q is an integer in [-127, 127] (|v| <= the row's absmax): q + 128 lands in its byte with one
      // v_cvt_pk_u8_f32, and flipping bit 7 of every byte turns the biased value into two's complement
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo = __builtin_amdgcn_cvt_pk_u8_f32(q[e] + 128.0f, (uint32_t)e, lo);
        hi = __builtin_amdgcn_cvt_pk_u8_f32(q[e + 4] + 128.0f, (uint32_t)e, hi);
      }
      lo ^= 0x80808080u;
      hi ^= 0x80808080u;
      if (a.codes_rm) *reinterpret_cast<uint2*>(a.codes_rm + (size_t)m * a.K + k0) = make_uint2(lo, hi);
    }
    if (a.xq_packed && p >= 0)
      *reinterpret_cast<uint2*>(a.xq_packed + packed_offset((uint32_t)p, k0, a.KB)) = make_uint2(lo, hi);
  }
}

// ---------------------------------------------------------------------------------------
// LoRA A re-layout: A [n, K, r] (rank contiguous) -> At [n, r, K] (K contiguous), so that an
// MFMA operand (8 consecutive k of one rank column) is one 16-byte load.  LoRA parameters
// are trainable and may change between calls, so this runs per call; it moves n*K*r*2 bytes.
// ---------------------------------------------------------------------------------------
__device__ inline void lora_a_transpose_item(const uint16_t* __restrict__ a, uint16_t* __restrict__ at,
                                             uint32_t n_groups, uint32_t K, uint32_t r, uint64_t idx) {
  const uint32_t rc = (r + 7u) / 8u;  // 8-wide rank chunks per k
  const uint64_t total = (uint64_t)n_groups * K * rc;
  if (idx >= total) return;
  const uint32_t ch = (uint32_t)(idx % rc);
  const uint64_t gk = idx / rc;  // group * K + k
  const uint32_t k = (uint32_t)(gk % K);
  const uint32_t grp = (uint32_t)(gk / K);
  const uint16_t* src = a + gk * r + ch * 8u;
  uint16_t v[8];
  if ((r & 7u) == 0) {
    const v8us w = *reinterpret_cast<const v8us*>(src);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = w[e];
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (ch * 8u + e < r) ? src[e] : (uint16_t)0;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t col = ch * 8u + e;
    if (col < r) at[((size_t)grp * r + col) * K + k] = v[e];
  }
}

// ---------------------------------------------------------------------------------------
// LoRA B re-layout: B [n, r, N] -> MFMA B-operand order bp[n][N_pad/32][nkk][64 lanes][8]:
// lane (c = l % 32, h = l / 32) of packed column block cb holds rows 16 kk + 8 h + 0..7 (zero
// beyond the rank) of the original column packed_to_orig_col(32 cb + c) (zero beyond N).
// Like A^T this runs per call because LoRA parameters are trainable.
// ---------------------------------------------------------------------------------------
__device__ inline void lora_b_pack_item(const uint16_t* __restrict__ b, unsigned char* __restrict__ bp,
                                        uint32_t n_groups, uint32_t r, uint32_t N, uint32_t ncb, uint32_t nkk,
                                        uint64_t idx) {
  const uint64_t total = (uint64_t)n_groups * ncb * nkk * 64u;  // one 16-byte operand per thread
  if (idx >= total) return;
  const uint32_t l = (uint32_t)(idx & 63u);
  const uint64_t rest = idx >> 6;
  const uint32_t kk = (uint32_t)(rest % nkk);
  const uint64_t gc = rest / nkk;
  const uint32_t cb = (uint32_t)(gc % ncb), grp = (uint32_t)(gc / ncb);
  const uint32_t col = packed_to_orig_col(cb * 32u + (l & 31u));
  v8us o = {0, 0, 0, 0, 0, 0, 0, 0};
  if (col < N) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t row = 16u * kk + 8u * (l >> 5) + e;
      if (row < r) o[e] = b[((size_t)grp * r + row) * N + col];
    }
  }
  *reinterpret_cast<v8us*>(bp + idx * 16u) = o;
}

// ---------------------------------------------------------------------------------------
// LoRA A re-layout for the dense path's quantizer: A [n, K, r] -> the B-operand order of
// v_mfma_f32_16x16x32_bf16, ap[n][K_pad/32][nkk][64 lanes][8]: lane (i = l % 16, q = l / 16) of
// k-block kb and rank block b holds k = 32 kb + 8 q + 0..7 (zero beyond K) of rank column
// 16 b + i (zero beyond the rank).  A wave's operand load is then 1 KiB of consecutive memory
// (eight cache lines) where the transposed layout gives it sixteen half-used lines, and the
// quantizer's LoRA-A step is bound by the cache lines its loads touch.
// ---------------------------------------------------------------------------------------
__device__ inline void lora_a_pack_item(const uint16_t* __restrict__ a, unsigned char* __restrict__ ap,
                                        uint32_t n_groups, uint32_t K, uint32_t r, uint32_t KB, uint32_t nkk,
                                        uint64_t idx) {
  const uint64_t total = (uint64_t)n_groups * KB * nkk * 64u;  // one 16-byte operand per thread
  if (idx >= total) return;
  const uint32_t l = (uint32_t)(idx & 63u);
  const uint64_t rest = idx >> 6;
  const uint32_t b = (uint32_t)(rest % nkk);
  const uint64_t gk = rest / nkk;
  const uint32_t kb = (uint32_t)(gk % KB), grp = (uint32_t)(gk / KB);
  const uint32_t col = 16u * b + (l & 15u);
  v8us o = {0, 0, 0, 0, 0, 0, 0, 0};
  if (col < r) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t k = 32u * kb + 8u * (l >> 4) + e;
      if (k < K) o[e] = a[((size_t)grp * K + k) * r + col];
    }
  }
  *reinterpret_cast<v8us*>(ap + idx * 16u) = o;
}

// The same for lora_a_kernel (v_mfma_f32_32x32x16_bf16, 64-wide k steps), whose operand loads of the
// transposed A touch 32 cache lines each:
// ap[n][ceil(K / 64)][RB][4][64 lanes][8]: lane (i = l % 32, h = l / 32) of k step s, rank block b and
// quarter t holds k = 64 s + 32 h + 8 t + 0..7 of rank column 32 b + i.  Pays with few adapters of many
// rows each; with 128 experts of rank 16 (padded to 32 columns, packed per call) it measured slower.
__device__ inline void lora_a_pack32_item(const uint16_t* __restrict__ a, unsigned char* __restrict__ ap,
                                          uint32_t n_groups, uint32_t K, uint32_t r, uint32_t n_steps, uint32_t rb,
                                          uint64_t idx) {
  const uint64_t total = (uint64_t)n_groups * n_steps * rb * 256u;  // one 16-byte operand per thread
  if (idx >= total) return;
  const uint32_t l = (uint32_t)(idx & 63u), t = (uint32_t)(idx >> 6) & 3u;
  const uint64_t rest = idx >> 8;
  const uint32_t b = (uint32_t)(rest % rb);
  const uint64_t gs = rest / rb;
  const uint32_t st = (uint32_t)(gs % n_steps), grp = (uint32_t)(gs / n_steps);
  const uint32_t col = 32u * b + (l & 31u);
  v8us o = {0, 0, 0, 0, 0, 0, 0, 0};
  if (col < r) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t k = 64u * st + 32u * (l >> 5) + 8u * t + e;
      if (k < K) o[e] = a[((size_t)grp * K + k) * r + col];
    }
  }
  *reinterpret_cast<v8us*>(ap + idx * 16u) = o;
}

// Clears `count` 32-bit words (one workgroup).
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* p, uint32_t count) {
  for (uint32_t i = threadIdx.x; i < count; i += 256u) p[i] = 0u;
}

// ---------------------------------------------------------------------------------------
// One launch for the three independent preparation jobs of a call: adapter routing (block 0
// when `idx` is given), LoRA A transposition and LoRA B operand packing (the other blocks).
// ---------------------------------------------------------------------------------------
struct LoraPrepArgs {
  const int32_t* idx;        // adapter per row, or null (no routing block)
  int32_t* src_row; int32_t* dst_pos; int32_t* slot_group; int32_t* blk_range;
  const uint16_t* lora_a;    // bf16 [n_groups, K, r]
  const uint16_t* lora_b;    // bf16 [n_groups, r, N]
  uint16_t* at;              // bf16 [n_groups, r, K]
  unsigned char* bp;         // packed B operands
  uint32_t M, K, N, n_groups, r, nkk, ncb, slots, route_blocks, a_blocks;
  uint32_t route_pad;        // dense routing block: every group's first slot is a multiple of this (0 or 1: packed)
  uint32_t a_operand_kb;     // 0: `at` is the transposed A; else K_pad / 32 and `at` takes A in MFMA operand order
  uint32_t a_operand_steps, a_operand_rb;  // or: ceil(K / 64) and the 32-wide rank blocks of lora_a_kernel's operand order
  // grouped (ragged) call: the routing block lays the groups out from their sizes instead
  const int32_t* group_sizes;  // int32 [n_groups] or null
  uint32_t group_pad;          // slots every group is padded to
  uint16_t* zero_out;          // bf16 [M, zero_cols]: rows beyond the groups are cleared, or null
  uint32_t zero_cols;
};

__global__ __launch_bounds__(1024) void lora_prep_kernel(LoraPrepArgs p) {
  uint32_t b = blockIdx.x;
  if (b < p.route_blocks) {
    if (p.group_sizes)
      route_groups_block(p.group_sizes, p.M, p.n_groups, p.slots, p.src_row, p.dst_pos, p.blk_range, p.group_pad,
                         p.zero_out, p.zero_cols, b, p.route_blocks);
    else
      route_rows_block(p.idx, p.M, p.n_groups, p.slots, p.src_row, p.dst_pos, p.slot_group, p.blk_range, nullptr, false,
                       p.route_pad > 1u ? p.route_pad : 1u);
    return;
  }
  b -= p.route_blocks;
  if (b < p.a_blocks) {
    if (p.a_operand_steps)
      lora_a_pack32_item(p.lora_a, reinterpret_cast<unsigned char*>(p.at), p.n_groups, p.K, p.r, p.a_operand_steps,
                         p.a_operand_rb, (uint64_t)b * 1024u + threadIdx.x);
    else if (p.a_operand_kb)
      lora_a_pack_item(p.lora_a, reinterpret_cast<unsigned char*>(p.at), p.n_groups, p.K, p.r, p.a_operand_kb, p.nkk,
                       (uint64_t)b * 1024u + threadIdx.x);
    else
      lora_a_transpose_item(p.lora_a, p.at, p.n_groups, p.K, p.r, (uint64_t)b * 1024u + threadIdx.x);
    return;
  }
  b -= p.a_blocks;
  lora_b_pack_item(p.lora_b, p.bp, p.n_groups, p.r, p.N, p.ncb, p.nkk, (uint64_t)b * 1024u + threadIdx.x);
}

// ---------------------------------------------------------------------------------------
// LoRA-A projection on bf16 MFMA: z[p, :] = n[src_row[p], :] @ A[group(p)]  (float32
// accumulation of exact bf16 products; skyrl/tx/kernels/quantized_lora.py:300-301 and
// skyrl/tx/layers/lora.py:150).  One workgroup of 8 waves per 32-row block; the waves take
// disjoint K ranges and are reduced through LDS in wave order.  The float32 result is split
// into three bf16 terms (z = hi + mid + lo exactly) and stored in the MFMA operand order the
// GEMM epilogue consumes: zp[block][kk][term][lane][8], lane = row % 32 + 32 * h holding the
// rank columns 16 kk + 8 h + 0..7.
// ---------------------------------------------------------------------------------------
struct LoraAArgs {
  const uint16_t* xsrc;     // bf16 [M, K] (x, or the normalized rows)
  const uint16_t* at;       // bf16 [n_groups, r, K], or A in operand order (lora_a_pack32_item) when at_operand is set
  uint32_t at_operand;      // 0 or 1
  const int32_t* src_row;   // or null (identity)
  const int32_t* slot_group;// or null (group 0)
  const int32_t* blk_range; // or null
  unsigned char* zp;        // packed z fragments
  uint32_t M, K, r, nkk, steps_per_wave, n_steps, n_blocks;
  uint32_t nterms;          // bf16 terms carried per value: 3 (exact split of the f32 value) or 2
  // Optional float32 copies (backward): zf = the raw projection, zsf = the projection times the
  // row's group scale; with group_scale the packed fragments carry the scaled value.  [slot][zf_stride]
  float* zf; float* zsf; const float* group_scale; uint32_t zf_stride;
  // K split (backward): with n_ksplit > 1 the grid holds n_ksplit workgroups per row block, each
  // sums its own range of k steps and writes zf + ksplit_index * zf_slice (floats); the caller adds
  // the slices.  0 or 1: one workgroup per row block.
  uint32_t n_ksplit, zf_slice;
  // Optional gather on the way in (see QuantArgs): source row = row_map[row] / row_div, clamped to row_limit
  const int32_t* row_map;
  uint32_t row_div, row_limit;
};

// STAGED (RB = 1, the transposed A; with or without the K split): the operands of a k step travel through 8 KiB of LDS
// per wave.  A register load of an MFMA operand touches 32 cache lines of 32 used bytes, which the
// vector memory path delivers at a third of the rate of whole lines; a direct-to-LDS load in which
// eight lanes fetch one 128-byte line (of a row of x, of a rank column of A) moves eight whole lines,
// and the operands are then read from LDS (line pieces XOR-swizzled by the row, so that eight lanes
// never share a bank).  Which wave adds which k step, and in which order, does not change.
constexpr uint32_t kLoraAStageBytes = 16u * 8192u;
template <int RB, bool STAGED = false>  // RB: number of 32-wide rank blocks (1 or 2)
__global__ __launch_bounds__(1024) void lora_a_kernel(LoraAArgs a) {
  static_assert(!STAGED || RB == 1, "the staged form holds one rank block");
  __shared__ float red[4][RB][16][64];
  __shared__ float zs[32][RB * 32 + 1];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t nks = a.n_ksplit > 1u ? a.n_ksplit : 1u;
  const uint32_t pb = blockIdx.x / nks, ks = blockIdx.x % nks;
  if (pb >= a.n_blocks) return;
  if (a.blk_range && a.blk_range[pb] < 0) return;  // block beyond the rows in use
  const uint32_t range = a.blk_range ? (uint32_t)a.blk_range[pb] : 0u;
  const uint32_t glo = range & 0xffffu, ghi = range >> 16;
  const uint32_t i = lane & 31u, h = lane >> 5;
  const uint32_t p = pb * 32u + i;
  int src = a.src_row ? a.src_row[p] : (int)p;
  if (src >= (int)a.M) src = -1;
  if (a.row_map && src >= 0) src = (int)mapped_row(a.row_map[src], a.row_div, a.row_limit);
  const uint32_t rowgrp = (a.slot_group && ghi > glo) ? (uint32_t)a.slot_group[p] : glo;
  const uint16_t* xr = a.xsrc + (size_t)(src < 0 ? 0 : src) * a.K;
  v16f acc[RB];
#pragma unroll
  for (int b = 0; b < RB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;
  const uint32_t slice_steps = (a.n_steps + nks - 1u) / nks;
  const uint32_t slice_end = (ks + 1u) * slice_steps < a.n_steps ? (ks + 1u) * slice_steps : a.n_steps;
  uint32_t s0 = ks * slice_steps + wave * a.steps_per_wave, s1 = s0 + a.steps_per_wave;
  if (s1 > slice_end) s1 = slice_end;
  if constexpr (STAGED) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char stage_lds[];
    unsigned char* const my = stage_lds + wave * 8192u;  // x lines at 0, A lines at 4096
    // lane l fetches, for j = 0..3, piece (l % 8) ^ (l / 8) of the 128-byte line of row / column 8 j + l / 8
    const uint32_t r8 = lane >> 3, piece = (lane & 7u) ^ r8;
    const uint16_t* xrow[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
      const uint32_t pj = pb * 32u + 8u * j + r8;
      int sj = a.src_row ? a.src_row[pj] : (int)pj;
      if (sj >= (int)a.M) sj = -1;
      if (a.row_map && sj >= 0) sj = (int)mapped_row(a.row_map[sj], a.row_div, a.row_limit);
      xrow[j] = a.xsrc + (size_t)(sj < 0 ? 0 : sj) * a.K;
    }
    // where lane (i, h) finds quarter t of its operand: line i, piece 4 h + t
    const uint32_t rd = (i >> 3) * 1024u + (i & 7u) * 128u;
    for (uint32_t grp = glo; grp <= ghi; ++grp) {
      const bool mine = src >= 0 && rowgrp == grp;
      const uint16_t* atg = a.at + (size_t)grp * a.r * a.K;
      for (uint32_t s = s0; s < s1; ++s) {
        uint32_t kp = s * 64u + piece * 8u;
        if (kp >= a.K) kp = 0;  // a piece beyond K: any address inside the row; it is zeroed where it is used
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
          load_1k_to_lds(reinterpret_cast<const unsigned char*>(xrow[j] + kp), my + j * 1024u);
        v8us xa[4], wb[4];
        if (a.at_operand) {  // kernel-uniform: A already lies in operand order (zero beyond K and the rank)
#pragma unroll
          for (uint32_t t = 0; t < 4; ++t)
            wb[t] = *(reinterpret_cast<const v8us*>(a.at) + (((size_t)grp * a.n_steps + s) * 4u + t) * 64u + lane);
        } else {
#pragma unroll
          for (uint32_t j = 0; j < 4; ++j) {
            uint32_t col = 8u * j + r8;
            if (col >= a.r) col = 0;
            load_1k_to_lds(reinterpret_cast<const unsigned char*>(atg + (size_t)col * a.K + kp), my + 4096u + j * 1024u);
          }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t) {
          const uint32_t off = rd + (((4u * h + t) ^ (i & 7u)) * 16u);
          const v8us zero = {0, 0, 0, 0, 0, 0, 0, 0};
          const bool ok = s * 64u + 32u * h + 8u * t < a.K;
          const v8us xv = *reinterpret_cast<const v8us*>(my + off);
          xa[t] = (mine && ok) ? xv : zero;
          if (!a.at_operand) {
            const v8us wv = *reinterpret_cast<const v8us*>(my + 4096u + off);
            wb[t] = (i < a.r && ok) ? wv : zero;
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the lines are read before the next step's loads land on them
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, xa[t]), __builtin_bit_cast(v8bf, wb[t]),
                                                           acc[0], 0, 0, 0);
      }
    }
  } else
  // A block at a group boundary runs once per group with the other groups' rows zeroed.
  for (uint32_t grp = glo; grp <= ghi; ++grp) {
    const bool mine = src >= 0 && rowgrp == grp;
    const uint16_t* atg = a.at + (size_t)grp * a.r * a.K;
    // U 64-wide k steps per iteration: all their operand loads go out before the MFMAs
    constexpr int U = RB == 1 ? 2 : 1;  // 1024 threads leave 128 registers per lane
    for (uint32_t s = s0; s < s1; s += U) {
      v8us xa[U][4], wb[U][RB][4];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t kbase = (s + u) * 64u + 32u * h;
        const bool step_ok = (s + u) < s1;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t k0 = kbase + 8u * t;
          const v8us zero = {0, 0, 0, 0, 0, 0, 0, 0};
          const bool ok = step_ok && k0 < a.K;
          xa[u][t] = (mine && ok) ? *reinterpret_cast<const v8us*>(xr + k0) : zero;
#pragma unroll
          for (int b = 0; b < RB; ++b) {
            const uint32_t col = b * 32u + i;
            if (a.at_operand)  // kernel-uniform: 1 KiB of consecutive memory per wave and load (zero beyond K and the rank)
              wb[u][b][t] = step_ok ? *(reinterpret_cast<const v8us*>(a.at) +
                                        ((((size_t)grp * a.n_steps + (s + u)) * RB + b) * 4u + t) * 64u + lane)
                                    : zero;
            else
              wb[u][b][t] = (col < a.r && ok) ? *reinterpret_cast<const v8us*>(atg + (size_t)col * a.K + k0) : zero;
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int b = 0; b < RB; ++b)
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, xa[u][t]),
                                                             __builtin_bit_cast(v8bf, wb[u][b][t]), acc[b], 0, 0, 0);
    }
  }
  // fixed-order reduction over the 16 waves: waves 4..7, 8..11, 12..15 are added, in that order,
  // onto waves 0..3, whose four partial sums are then added in wave order
  for (uint32_t round = 1; round < 4; ++round) {
    if ((wave >> 2) == round) {
#pragma unroll
      for (int b = 0; b < RB; ++b)
#pragma unroll
        for (int e = 0; e < 16; ++e) red[wave & 3u][b][e][lane] = acc[b][e];
    }
    __syncthreads();
    if (wave < 4) {
#pragma unroll
      for (int b = 0; b < RB; ++b)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[b][e] = acc[b][e] + red[wave][b][e][lane];
    }
    __syncthreads();
  }
  if (wave < 4) {
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) red[wave][b][e][lane] = acc[b][e];
  }
  __syncthreads();
  for (uint32_t q = threadIdx.x; q < RB * 1024u; q += 1024u) {
    const uint32_t l = q & 63u, e = (q >> 6) & 15u, b = q >> 10;
    float sum = red[0][b][e][l];
#pragma unroll
    for (int w = 1; w < 4; ++w) sum += red[w][b][e][l];
    zs[8u * (e >> 2) + 4u * (l >> 5) + (e & 3u)][b * 32u + (l & 31u)] = sum;
  }
  __syncthreads();
  if (a.zf || a.group_scale) {
    for (uint32_t q = threadIdx.x; q < 32u * RB * 32u; q += 1024u) {
      const uint32_t row = q / (RB * 32u), col = q % (RB * 32u);
      const float raw = zs[row][col];
      if (a.zf) a.zf[(size_t)ks * a.zf_slice + (size_t)(pb * 32u + row) * a.zf_stride + col] = raw;
      if (a.group_scale) {
        const uint32_t gr = (a.slot_group && ghi > glo) ? (uint32_t)a.slot_group[pb * 32u + row] : glo;
        const float scaled = raw * a.group_scale[gr];
        zs[row][col] = scaled;
        if (a.zsf) a.zsf[(size_t)(pb * 32u + row) * a.zf_stride + col] = scaled;
      }
    }
    __syncthreads();
  }
  if (!a.zp) return;
  for (uint32_t q = threadIdx.x; q < a.nkk * 3u * 64u; q += 1024u) {
    const uint32_t l = q & 63u, term = (q >> 6) % 3u, kk = q / 192u;
    const uint32_t row = l & 31u, hh = l >> 5;
    v8us o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float z = zs[row][16u * kk + 8u * hh + e];
      const uint32_t b0 = f32_to_bf16_bits(z);
      const float r1 = z - bf16_bits_to_f32(b0);
      const uint32_t b1 = f32_to_bf16_bits(r1);
      const float r2 = r1 - bf16_bits_to_f32(b1);
      const uint32_t b2 = f32_to_bf16_bits(r2);
      o[e] = (unsigned short)(term == 0 ? b0 : (term == 1 ? b1 : (a.nterms >= 3u ? b2 : 0u)));
    }
    *reinterpret_cast<v8us*>(a.zp + (((size_t)pb * a.nkk + kk) * 3u + term) * kBlockBytes + l * 16u) = o;
  }
}

// ---------------------------------------------------------------------------------------
// Quantizer and LoRA-A projection in one pass over x (the dense path's prologue).
// One workgroup of 16 waves per R grouped slots (R = 16, or 8 / 4 / 2 when longer rows would not fit the
// LDS: half a 32-row block or a part of one):
//   1. wave w < R copies slot row w from memory into the LDS with direct-to-LDS loads -- the only
//      time x is read -- and takes its statistics from there: (RMSNorm sum of squares, the row normalized
//      in place,) absmax -> scale;
//   2. the waves split K in 32-wide blocks; lane (i = lane % 16, q = lane / 16) takes the 8 (normalized)
//      values k = 32 kb + 8 q .. +7 of row i from the LDS and uses them twice: as int8 codes written into
//      the activation's 1 KiB fragment block, and as the A operand of v_mfma_f32_16x16x32_bf16 against the
//      LoRA A of the row's group in that instruction's operand order, so the normalized rows never travel
//      through memory;
//   3. the waves' z tiles are added in a fixed order, split exactly into three bf16 terms and
//      stored in the operand order the GEMM epilogue reads (see lora_a_kernel).
// Arithmetic follows quant_rows_kernel (skyrl/tx/kernels/quantized_lora.py:199-212 and the
// RMSNorm of bf16_rms_gate_up_lora_swiglu.py:299-303) operation for operation.
// ---------------------------------------------------------------------------------------
struct QuantLoraArgs {
  const uint16_t* x;        // bf16 [M, K]
  const float* gamma;       // f32 [K] (RMS only)
  float eps;
  uint32_t M, K, K_pad, KB, n_half_blocks;  // n_half_blocks = ceil(M / 16)
  const int32_t* src_row;   // original row of a slot, or null (identity)
  const int32_t* slot_group;// or null
  const int32_t* blk_range; // per 32-slot block, or null (group 0)
  unsigned char* xq_packed; // packed codes [slots/32][KB][1 KiB]
  float* sx_slots;          // f32 [slots]
  int8_t* codes_rm;         // row-major codes [M, K] or null
  float* scales_rm;         // f32 [M] or null
  uint16_t* xn_aux;         // bf16 [M, K] normalized rows for the caller, or null
  const uint16_t* at;       // LoRA A in MFMA operand order [n_groups][KB][CB][64 lanes][8 bf16] (lora_a_pack_item) or null (CB == 0)
  unsigned char* zp;        // packed z fragments
  uint32_t r, nkk, nterms;
  uint32_t* tile_ctr;       // 256 words cleared for the GEMM launches' tile counters, or null
  // Routing inside this launch (route_idx != null; M <= kInlineRouteMaxRows): every workgroup sorts the
  // adapter indices for itself and WRITES its slots' entries of src_row / slot_group / blk_range
  // (then non-const outputs, read later by the GEMM) instead of reading them.
  const int32_t* route_idx; // adapter per row
  uint32_t n_groups, slots;
  uint32_t group_pad;       // every group's first slot is a multiple of this (1: groups packed; 32: no block holds two groups)
  uint32_t rows_per_wg;     // R: 16, 8, 4 or 2 slots per workgroup (quant_lora_rows_per_wg)
  uint32_t row_stride;      // bytes between two rows in the LDS (quant_lora_row_stride)
};

constexpr uint32_t kInlineRouteMaxRows = 8192;  // eight rows per thread of a 1024-thread workgroup

// LDS bytes of a row: its 2 K bytes rounded up to the 1 KiB a wave's direct-to-LDS load moves, plus 16 so
// that the sixteen rows a wave reads side by side in step 2 (16 bytes each) fall on sixteen different
// bank groups.
__host__ __device__ inline uint32_t quant_lora_row_stride(uint32_t k) { return round_up(2u * k, 1024u) + 16u; }
constexpr uint32_t kQuantLoraLdsBudget = 150u * 1024u;  // rows + reduction tiles; the rest of the 160 KiB is static
__host__ __device__ inline uint32_t quant_lora_rows_per_wg(uint32_t k) {
  uint32_t r = 16u;
  while (r > 2u && r * quant_lora_row_stride(k) > kQuantLoraLdsBudget) r >>= 1;
  return r;
}
// dynamic LDS of a launch: the rows, or the reduction tiles that reuse the same bytes once the rows are spent
__host__ __device__ inline uint32_t quant_lora_lds_bytes(uint32_t k, uint32_t cb) {
  const uint32_t rows = quant_lora_rows_per_wg(k) * quant_lora_row_stride(k);
  const uint32_t red = 8u * (cb ? cb : 1u) * 4u * 64u * 4u;
  return rows > red ? rows : red;
}

// The routing tables of route_rows_block for the 16 slots [16 hb, 16 hb + 16), computed by the
// workgroup itself: rows keep their order inside a group (slot start[g] + j holds the j-th row of group
// g), which every workgroup derives alike from the adapter indices alone.  Returns through LDS:
// out_src[16], out_grp[16], out_range (the group range of the 32-slot block that holds the slots).
// With group_pad = 32 every group starts on a block boundary (the slots between a group's last row and
// the next group's first stay empty, src -1), so no 32-slot block holds rows of two groups: neither
// this kernel nor the GEMM's epilogue then runs a block once per group.  The slots in use end at
// sum(round_up(count, group_pad)) <= M + (group_pad - 1) * min(n_groups, M).
// Steps: every wave counts its rows per group (LDS atomics on its own counters: with 16 waves on a CU
// the vector ALU's share per wave makes a ballot per group and row several times dearer); wave 0 turns
// the counts into per-wave prefixes, the groups' first slots and the groups of the sixteen slots; the
// waves that hold the wanted ranks of a group pick their rows.  Three barriers.
__device__ inline void route_rows_inline(const int32_t* __restrict__ idx, uint32_t M, uint32_t n_groups,
                                         uint32_t slots, uint32_t group_pad, uint32_t hb, int* out_src, int* out_grp,
                                         uint32_t* out_range, int* out_last_group) {
  __shared__ int wcnt[kMaxAdapters][17];  // rows of group g in wave w; then the exclusive prefix over the waves
  __shared__ int start[kMaxAdapters + 1];
  __shared__ int cnt[kMaxAdapters];
  __shared__ uint32_t used_end;  // first slot behind the last group
  __shared__ int g_first_s, g_last_s;
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t per = (M + 1023u) / 1024u;  // consecutive rows per thread (<= 8)
  int mine[8];
#pragma unroll
  for (uint32_t j = 0; j < 8; ++j) {
    const uint32_t i = tid * per + j;
    int a = -1;
    if (j < per && i < M) {
      a = idx[i];
      a = a < 0 ? 0 : (a >= (int)n_groups ? (int)n_groups - 1 : a);
    }
    mine[j] = a;
  }
  if (lane < n_groups) wcnt[lane][wave] = 0;  // (the loads above are still in flight)
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (uint32_t j = 0; j < 8; ++j)
    if (j < per && mine[j] >= 0) atomicAdd(&wcnt[mine[j]][wave], 1);  // integer counts of one wave: any order
  __syncthreads();
  const uint32_t p0 = hb * 16u;
  if (wave == 0) {  // lane g: group g (n_groups <= 64)
    int total = 0;
    if (lane < n_groups) {
      int c[16];
#pragma unroll
      for (uint32_t w = 0; w < 16; ++w) c[w] = wcnt[lane][w];  // all reads first: one round trip
#pragma unroll
      for (uint32_t w = 0; w < 16; ++w) {
        wcnt[lane][w] = total;
        total += c[w];
      }
    }
    const int padded = (int)round_up((uint32_t)total, group_pad);
    int incl = padded;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off, 64);
      if ((int)lane >= off) incl += up;
    }
    const int st = incl - padded;  // first slot of group `lane`
    const uint32_t E = (uint32_t)__shfl(incl, 63, 64);
    const unsigned long long nonempty = __builtin_amdgcn_ballot_w64(total > 0);
    const int last_ne = nonempty ? 63 - __builtin_clzll(nonempty) : 0;
    if (lane < n_groups) { start[lane] = st; cnt[lane] = total; }
    if (lane == 0) { start[n_groups] = (int)E; used_end = E; *out_last_group = last_ne; }
    // group of a slot: the last group whose first slot is not behind it (empty groups share their
    // successor's first slot, so the last one is the one that holds the slot); slots behind the last
    // group follow the last non-empty one
    auto group_of = [&](uint32_t p) -> int {
      if (p >= E) return last_ne;
      const unsigned long long m = __builtin_amdgcn_ballot_w64(lane < n_groups && (uint32_t)st <= p);
      return m ? 63 - __builtin_clzll(m) : 0;
    };
    const uint32_t p_end = (p0 + 16u < E) ? p0 + 16u : E;
    const int gf = group_of(p0), gl = group_of(p_end ? p_end - 1u : 0u);
    int my_grp = group_of(p0 + 15u);  // (the slots behind the last group follow the last non-empty one)
    if (my_grp != gf) {  // wave-uniform: the sixteen slots hold a group boundary (or the end)
#pragma unroll
      for (uint32_t s16 = 0; s16 < 16; ++s16) {
        const int g = group_of(p0 + s16);
        if (lane == s16) my_grp = g;
      }
    }
    if (lane < 16u) { out_grp[lane] = my_grp; out_src[lane] = -1; }
    const uint32_t b0 = (p0 / 32u) * 32u;
    const uint32_t b1 = (b0 + 31u < E) ? b0 + 31u : (E ? E - 1u : 0u);
    const int gb0 = group_of(b0), gb1 = group_of(b1);
    if (lane == 0) {
      *out_range = b0 >= E ? 0u : ((uint32_t)gb0 | ((uint32_t)gb1 << 16));
      g_first_s = p0 < E ? gf : 1;  // an empty range when the slots lie behind the last group
      g_last_s = p0 < E ? gl : 0;
    }
  }
  __syncthreads();
  // the rows of the slots in use, group by group (a workgroup's 16 slots usually lie in one group)
  const uint32_t E = used_end;
  const uint32_t p_end = (p0 + 16u < E) ? p0 + 16u : E;
  const int g_first = g_first_s, g_last = g_last_s;
  for (int g = g_first; g <= g_last; ++g) {  // workgroup-uniform
    const int cg = cnt[g], sg = start[g];
    if (cg == 0) continue;
    // slots of group g among mine: ranks [lo, hi)
    const int lo = ((int)p0 > sg ? (int)p0 : sg) - sg;
    const int hi = ((int)p_end < sg + cg ? (int)p_end : sg + cg) - sg;
    const int wbefore = wcnt[g][wave];
    const int wafter = wave < 15u ? wcnt[g][wave + 1u] : cg;
    if (hi <= lo || wafter <= lo || wbefore >= hi) continue;  // wave-uniform: none of the wanted ranks is in this wave
    int c = 0;
#pragma unroll
    for (uint32_t j = 0; j < 8; ++j) c += (mine[j] == g) ? 1 : 0;
    int incl = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off, 64);
      if ((int)lane >= off) incl += up;
    }
    int rank = wbefore + incl - c;
#pragma unroll
    for (uint32_t j = 0; j < 8; ++j) {
      if (mine[j] == g) {
        if (rank >= lo && rank < hi) out_src[sg + rank - (int)p0] = (int)(tid * per + j);
        ++rank;
      }
    }
  }
  __syncthreads();
}

template <int CB, bool RMS>  // CB: 16-wide rank blocks (0 = no LoRA, 1, 2, 4)
__global__ __launch_bounds__(1024) void quant_lora_kernel(QuantLoraArgs a) {
  constexpr int kCB = CB > 0 ? CB : 1;
  extern __shared__ __attribute__((aligned(1024))) unsigned char ql_lds[];  // the rows; later the wave tiles of z
  __shared__ float row_scale[16];
  __shared__ int row_src[16];
  __shared__ float zs[16][kCB * 16 + 1];
  typedef float red_t[kCB][4][64];  // wave tiles on their way to waves 0..7, then 0..3
  red_t* const red = reinterpret_cast<red_t*>(ql_lds);
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t R = a.rows_per_wg, per_hb = 16u / R;
  const uint32_t hb = blockIdx.x / per_hb;           // half block: slots 16 hb .. 16 hb + 15
  const uint32_t r0 = (blockIdx.x % per_hb) * R;     // this workgroup's slots inside it: r0 .. r0 + R - 1
  if (a.tile_ctr && blockIdx.x == 0 && tid < 256u) a.tile_ctr[tid] = 0u;
  if (hb >= a.n_half_blocks) return;
  const uint32_t pb = hb >> 1, half16 = hb & 1u;
  __shared__ int route_src[16], route_grp[16], route_last_group;
  __shared__ uint32_t route_range;
  const bool route_here = a.route_idx != nullptr;  // workgroup-uniform
  if (route_here) {
    route_rows_inline(a.route_idx, a.M, a.n_groups, a.slots, a.group_pad, hb, route_src, route_grp, &route_range,
                      &route_last_group);
    // the tables the GEMM reads later (every workgroup of a half block derives the same values)
    if (tid >= r0 && tid < r0 + R) {
      const_cast<int32_t*>(a.src_row)[hb * 16u + tid] = route_src[tid];
      const_cast<int32_t*>(a.slot_group)[hb * 16u + tid] = route_grp[tid];
    }
    if (tid == 16u) const_cast<int32_t*>(a.blk_range)[pb] = (int32_t)route_range;  // (the same value from each)
    if (blockIdx.x + 1u == gridDim.x) {  // the padding slots behind the last 32-row block, up to the GEMM's tile rows
      for (uint32_t p = a.n_half_blocks * 16u + tid; p < a.slots; p += 1024u) {
        const_cast<int32_t*>(a.src_row)[p] = -1;
        const_cast<int32_t*>(a.slot_group)[p] = route_last_group;
        if ((p & 31u) == 0) const_cast<int32_t*>(a.blk_range)[p / 32u] = 0;
      }
    }
  }
  if (a.group_pad > 1u && (route_here || a.src_row)) {
    // padded groups leave whole stretches of slots empty: nothing reads their codes, scales or z
    int any = 0;
    for (uint32_t j = r0; j < r0 + R; ++j) any |= ((route_here ? route_src[j] : a.src_row[hb * 16u + j]) >= 0) ? 1 : 0;
    if (!any) return;  // workgroup-uniform
  }
  // ---- 1. the rows into the LDS and their statistics: wave w, slot row r0 + w
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)ql_lds;
  const uint32_t row_bytes = 2u * a.K;
  const uint32_t n_chunks = (row_bytes + 1023u) / 1024u;  // 1 KiB pieces of a row (the last one may be partial)
  if (wave < R) {
    const uint32_t sl = r0 + wave;
    const uint32_t p = hb * 16u + sl;
    int src = route_here ? route_src[sl] : (a.src_row ? a.src_row[p] : (int)p);
    if (src < 0 || src >= (int)a.M) src = -1;
    src = __builtin_amdgcn_readfirstlane(src);
    unsigned char* const rowl = ql_lds + wave * a.row_stride;
    float inv = 1.0f;
    uint32_t amax_bits = 0;  // largest |value| as bf16 bits in both halves
    if (src >= 0) {
      const unsigned char* xr = reinterpret_cast<const unsigned char*>(a.x) + (size_t)src * row_bytes;
      const uint32_t row_lds = lds_addr + wave * a.row_stride;
      for (uint32_t u = 0; u < n_chunks; ++u) {
        const uint32_t voff = u * 1024u + lane * 16u;
        if (voff < row_bytes) lds_load_1k(xr, voff, row_lds + u * 1024u);
      }
      // (the first chunk's norm weights travel with the row)
      float4 gn0 = make_float4(0.f, 0.f, 0.f, 0.f), gn1 = gn0;
      if (RMS && lane * 16u < row_bytes) {
        gn0 = *reinterpret_cast<const float4*>(a.gamma + lane * 8u);
        gn1 = *reinterpret_cast<const float4*>(a.gamma + lane * 8u + 4);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (RMS) {
        double ss = 0.0;
        for (uint32_t u = 0; u < n_chunks; ++u) {
          const uint32_t off = u * 1024u + lane * 16u;
          const uint4 raw = off < row_bytes ? *reinterpret_cast<const uint4*>(rowl + off) : make_uint4(0, 0, 0, 0);
          const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // the square of a bf16 value is exact in double, so the fused form rounds like mul + add
            const double lo = (double)__uint_as_float(w[e] << 16), hi = (double)__uint_as_float(w[e] & 0xffff0000u);
            ss = __builtin_fma(lo, lo, ss);
            ss = __builtin_fma(hi, hi, ss);
          }
        }
        ss = wave_sum(ss);
        const float var = (float)(ss / (double)a.K);
        inv = 1.0f / sqrtf(var + a.eps);
      }
      for (uint32_t u = 0; u < n_chunks; ++u) {
        const uint32_t off = u * 1024u + lane * 16u;
        float4 g0 = gn0, g1 = gn1;
        if (RMS) {  // the norm weights of the next chunk are requested before this one is worked on
          const uint32_t offn = off + 1024u;
          if (offn < row_bytes) {
            gn0 = *reinterpret_cast<const float4*>(a.gamma + (offn >> 1));
            gn1 = *reinterpret_cast<const float4*>(a.gamma + (offn >> 1) + 4);
          }
        }
        if (off >= row_bytes) continue;
        uint4 raw = *reinterpret_cast<const uint4*>(rowl + off);
        if (RMS) {
          const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
          uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float t0 = __uint_as_float(w[e] << 16) * inv, t1 = __uint_as_float(w[e] & 0xffff0000u) * inv;
            t0 = t0 * g[2 * e];
            t1 = t1 * g[2 * e + 1];
            w[e] = pack_bf16x2(t0, t1);
          }
          raw = make_uint4(w[0], w[1], w[2], w[3]);
          *reinterpret_cast<uint4*>(rowl + off) = raw;  // the normalized row replaces the row
          if (a.xn_aux) *reinterpret_cast<uint4*>(reinterpret_cast<unsigned char*>(a.xn_aux) + (size_t)src * row_bytes + off) = raw;
        }
        // |bf16| compares like its 15 magnitude bits as an integer (a NaN ends above every number and the
        // scale then falls back to 1, as the reference's comparison amax > 0 does)
        const uint32_t m0 = raw.x & 0x7fff7fffu, m1 = raw.y & 0x7fff7fffu, m2 = raw.z & 0x7fff7fffu, m3 = raw.w & 0x7fff7fffu;
        typedef unsigned short us2 __attribute__((ext_vector_type(2)));
        us2 mx = __builtin_bit_cast(us2, amax_bits);
        mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, m0));
        mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, m1));
        mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, m2));
        mx = __builtin_elementwise_max(mx, __builtin_bit_cast(us2, m3));
        amax_bits = __builtin_bit_cast(uint32_t, mx);
      }
    }
    uint32_t top = (amax_bits >> 16) > (amax_bits & 0xffffu) ? (amax_bits >> 16) : (amax_bits & 0xffffu);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t other = (uint32_t)__shfl_xor((int)top, o, 64);
      top = other > top ? other : top;
    }
    const float amax = __uint_as_float(top << 16);
    const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    if (lane == 0) {
      row_scale[sl] = scale;
      row_src[sl] = src;
      a.sx_slots[p] = scale;
      if (a.scales_rm && src >= 0) a.scales_rm[src] = scale;
    }
  }
  __syncthreads();

  // ---- 2. codes and z
  const uint32_t i = lane & 15u, q = lane >> 4;
  const bool mine_row = i >= r0 && i < r0 + R;  // slot row i belongs to this workgroup
  const int src = mine_row ? row_src[i] : -1;
  const float scale = mine_row ? row_scale[i] : 1.0f;
  const float rscale = __builtin_amdgcn_rcpf(scale);
  const unsigned char* const rowl = ql_lds + (mine_row ? i - r0 : 0u) * a.row_stride;
  const uint32_t range = CB == 0 ? 0u : (route_here ? route_range : (a.blk_range ? (uint32_t)a.blk_range[pb] : 0u));
  const uint32_t glo = range & 0xffffu, ghi = range >> 16;
  const uint32_t rowgrp = (CB > 0 && ghi > glo)
                              ? (route_here ? (uint32_t)route_grp[i] : (a.slot_group ? (uint32_t)a.slot_group[hb * 16u + i] : glo))
                              : glo;
  v4f acc[kCB];
#pragma unroll
  for (int b = 0; b < kCB; ++b) acc[b] = v4f{0.f, 0.f, 0.f, 0.f};
  // fragment block byte offset of this lane's 8 codes: row 16*half16 + i, k half q/2, byte 8*(q%2)
  const uint32_t code_off = (16u * half16 + i + 32u * (q >> 1)) * 16u + 8u * (q & 1u);
  // One pass over the k-blocks per group present among the slots (one, except at a group boundary): the
  // first pass also forms the codes; a later pass only adds the rows of its group to z (the rows are still
  // in the LDS).  The loop is kept rolled, two k-blocks per trip with their operands requested one trip
  // ahead and no load inside the work on a k-block, so that the compiler's waits count loads instead of
  // draining them.
  auto request = [&](uint32_t grp, uint32_t kb, v4i (&w)[kCB], uint4& raw) {
    if constexpr (CB > 0) {
      // operands of group grp, k-block kb: CB consecutive 1 KiB pieces (zero beyond K and the rank)
      const v4i* ap = reinterpret_cast<const v4i*>(a.at) + (((size_t)grp * a.KB + kb) * CB) * 64u + lane;
#pragma unroll
      for (int b = 0; b < CB; ++b) w[b] = kb < a.KB ? ap[b * 64] : v4i{0, 0, 0, 0};
    }
    const uint32_t k0 = kb * 32u + q * 8u;
    raw = (kb < a.KB && k0 < a.K && src >= 0) ? *reinterpret_cast<const uint4*>(rowl + 2u * k0) : make_uint4(0, 0, 0, 0);
  };
  auto work = [&](bool first, bool in_group, uint32_t kb, const v4i (&w)[kCB], const uint4& raw) {
    if (first) {  // wave-uniform
      const uint32_t k0 = kb * 32u + q * 8u;
      const bool live = src >= 0 && k0 < a.K;  // K is a multiple of 8
      const uint32_t nb[4] = {raw.x, raw.y, raw.z, raw.w};  // the (normalized) values as bf16 pairs
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = (e & 1) ? __uint_as_float(nb[e >> 1] & 0xffff0000u) : __uint_as_float(nb[e >> 1] << 16);
      // codes = rint(v / scale) with the correctly rounded quotient.  v * (1 / scale) with the
      // hardware reciprocal is within 3 * 2^-24 * 128 < 2.3e-5 of it, so both round to the same
      // integer unless the product lies that close to a tie; those cases (and scales outside the
      // reciprocal's safe range) are redone with the division.
      // The codes are formed biased by 128 (the fused v * (1 / scale) + 128 adds at most another 2^-17 to
      // the distance above, still far inside the tie margin): c is then an integer in [1, 255] (|v| <= the
      // row's absmax, so the clip of the reference never acts), lands in its byte with one
      // v_cvt_pk_u8_f32, and flipping bit 7 of every byte turns the biased value into two's complement.
      float c[8];
      float off_integer = 0.0f;  // largest distance of a quotient from its rounded value
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float t = __builtin_fmaf(v[e], rscale, 128.0f);
        c[e] = rintf(t);
        off_integer = fmaxf(off_integer, fabsf(t - c[e]));
      }
      const bool redo = !(scale > 1e-30f && scale < 1e30f) || off_integer > 0.49996f;  // margin 4e-5 > 2.3e-5 + 2^-17
      if (__builtin_amdgcn_ballot_w64(redo) != 0) {  // wave-uniform
#pragma unroll
        for (int e = 0; e < 8; ++e) c[e] = rintf(v[e] / scale) + 128.0f;
      }
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo = __builtin_amdgcn_cvt_pk_u8_f32(c[e], (uint32_t)e, lo);
        hi = __builtin_amdgcn_cvt_pk_u8_f32(c[e + 4], (uint32_t)e, hi);
      }
      lo ^= 0x80808080u;  // (a lane without a value holds zeros: 0 -> 128 -> code 0)
      hi ^= 0x80808080u;
      if (live && a.codes_rm) *reinterpret_cast<uint2*>(a.codes_rm + (size_t)src * a.K + k0) = make_uint2(lo, hi);
      if (mine_row) *reinterpret_cast<uint2*>(a.xq_packed + ((size_t)pb * a.KB + kb) * kBlockBytes + code_off) = make_uint2(lo, hi);
    }
    if constexpr (CB > 0) {
      // (zeros where the lane has no value; at a group boundary the rows of the other groups are zeroed)
      const v4i xa = in_group ? v4i{(int)raw.x, (int)raw.y, (int)raw.z, (int)raw.w} : v4i{0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < CB; ++b)
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, xa), __builtin_bit_cast(v8bf, w[b]),
                                                         acc[b], 0, 0, 0);
    }
  };
#pragma unroll 1
  for (uint32_t grp = glo; grp <= ghi; ++grp) {  // workgroup-uniform: one trip except at a group boundary
    const bool first = grp == glo;
    const bool in_group = ghi == glo || rowgrp == grp;
    v4i wa[kCB], wb2[kCB];
    uint4 ra, rb;
    request(grp, wave, wa, ra);
    request(grp, wave + 16u, wb2, rb);
#pragma unroll 1
    for (uint32_t kb = wave; kb < a.KB; kb += 32u) {
      work(first, in_group, kb, wa, ra);
      request(grp, kb + 32u, wa, ra);
      if (kb + 16u >= a.KB) break;  // wave-uniform
      work(first, in_group, kb + 16u, wb2, rb);
      request(grp, kb + 48u, wb2, rb);
    }
    if constexpr (CB == 0) break;
  }
  if constexpr (CB == 0) return;

  // ---- 3. fixed-order sum of the 16 wave tiles: 8..15 onto 0..7, 4..7 onto 0..3, then 0+1+2+3
  __syncthreads();  // the rows are spent: their bytes take the wave tiles
#pragma unroll 1
  for (uint32_t half = 8u; half >= 4u; half >>= 1) {
    if (wave >= half && wave < 2u * half) {
#pragma unroll
      for (int b = 0; b < kCB; ++b)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[wave - half][b][e][lane] = acc[b][e];
    }
    __syncthreads();
    if (wave < half) {
#pragma unroll
      for (int b = 0; b < kCB; ++b)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[b][e] = acc[b][e] + red[wave][b][e][lane];
    }
    __syncthreads();
  }
  if (wave < 4u) {
#pragma unroll
    for (int b = 0; b < kCB; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave][b][e][lane] = acc[b][e];
  }
  __syncthreads();
  // MFMA result layout: lane l holds column l % 16 and rows 4 * (l / 16) + e
  for (uint32_t t = tid; t < (uint32_t)kCB * 256u; t += 1024u) {
    const uint32_t l = t & 63u, e = (t >> 6) & 3u, b = t >> 8;
    const float sum = ((red[0][b][e][l] + red[1][b][e][l]) + red[2][b][e][l]) + red[3][b][e][l];
    zs[4u * (l >> 4) + e][b * 16u + (l & 15u)] = sum;
  }
  __syncthreads();
  // zp[pb][kk][term][lane64][8]: lane = row % 32 + 32 * hh holds rank columns 16 kk + 8 hh + 0..7
  for (uint32_t t = tid; t < a.nkk * 3u * 32u; t += 1024u) {
    const uint32_t row = t & 15u, hh = (t >> 4) & 1u, term = (t >> 5) % 3u, kk = t / 96u;
    if (row < r0 || row >= r0 + R) continue;
    v8us o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t col = 16u * kk + 8u * hh + e;
      const float z = col < (uint32_t)kCB * 16u ? zs[row][col] : 0.0f;
      const uint32_t b0 = f32_to_bf16_bits(z);
      const float r1 = z - bf16_bits_to_f32(b0);
      const uint32_t b1 = f32_to_bf16_bits(r1);
      const float r2 = r1 - bf16_bits_to_f32(b1);
      const uint32_t b2 = f32_to_bf16_bits(r2);
      o[e] = (unsigned short)(term == 0 ? b0 : (term == 1 ? b1 : (a.nterms >= 3u ? b2 : 0u)));
    }
    const uint32_t l64 = 16u * half16 + row + 32u * hh;
    *reinterpret_cast<v8us*>(a.zp + (((size_t)pb * a.nkk + kk) * 3u + term) * kBlockBytes + l64 * 16u) = o;
  }
}

}  // namespace w8a8
