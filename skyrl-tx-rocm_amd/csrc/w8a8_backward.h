// Backward of the W8A8 LoRA linear: the W8A16 input pull-back and the LoRA cotangents.
//   dx  = dy @ bf16(codes * sw).T  +  rs @ A[g].T          rs = (dy @ B[g].T) * s[g]
//   dA[g] = x_g.T @ rs_g      dB[g] = ((x_g @ A[g]).T @ dy_g) * s[g]      ds[g] = sum(dy_g * ((x_g @ A[g]) @ B[g]))
// Equations: skyrl/tx/kernels/quantized_lora.py:337-394.  The frozen weight enters the pull-back
// as bf16(codes * scales) per element with float32 accumulation of bf16 products, the policy of
// the reference's ROCm kernel (skyrl/tx/kernels/rocm/w8a8_lora.py:298-339); the LoRA terms stay in
// float32 and every cotangent is cast once.
//
// The packed weight keeps 16 consecutive k of one output column n in a lane; the pull-back
// contracts over n, so every 32 x 32 byte block is transposed on the matrix core itself:
// v_mfma_i32_32x32x32_i8 of the block against an identity operand returns W[n][k] with lane = k and
// sixteen n per lane, exactly the B operand of v_mfma_f32_32x32x16_bf16 once the integers are
// scaled and rounded to bf16.  No transposed ("shadow") copy of the weight exists.
#pragma once
#include "w8a8_device.h"
#include "w8a8_prologue.h"

namespace w8a8 {

// ---------------------------------------------------------------------------------------
// dy in MFMA A-operand order: dyp[row block][n block][q][64 lanes][8 bf16] (1 KiB per (block, q)).
// Lane (i = l % 32, h = l / 32) element e of (n block nb, q) holds packed weight column
//   32 nb + 16 q + 8 (e / 4) + 4 h + e % 4,
// the n that the transposing MFMA leaves in contraction slot 8 h + e of its q-th half.  Rows are
// in grouped (adapter-sorted) slot order; slots without a row and columns beyond N are zero.
// A wave takes a row block and a 128-column group at a time: a lane reads 4 x 16 consecutive
// original columns of its row and owns the pieces of the eight packed blocks (q, j = column % 4)
// that interleave them.
// The same pass computes r = dy @ B[group].T on bf16 MFMAs (the 8-value pieces a lane has loaded
// are A operands as they are; the matching pieces of B are 16-byte loads), so dy is read once:
// a workgroup of four waves owns one 32-row block and one slice of the 128-column groups, and
// leaves its partial sum in rpart[slice][slot][64]; bwd_r_finish_kernel adds the slices.
// ---------------------------------------------------------------------------------------
constexpr uint32_t kBwdRankStride = 64;  // floats per slot in the z / r tables
constexpr uint32_t kBwdChunkRows = 512;  // rows of a chunk of the LoRA cotangents
constexpr uint32_t kBwdStageRows = 256;  // rows whose skinny operand sits in LDS at a time

struct BwdPackDyArgs {
  const uint16_t* dy;        // bf16 [M, N]
  const int32_t* src_row;    // original row of a slot or null (identity)
  const int32_t* slot_group; // or null (group 0)
  const int32_t* blk_range;  // or null
  unsigned char* dyp;
  const uint16_t* lora_b;    // bf16 [n_groups, r, N] or null (no LoRA: packing only)
  float* rpart;              // f32 [n_slices][slots][64]
  uint32_t M, N, NB, n_row_blocks, n_col_groups, n_slices, groups_per_slice, r, slots;
};

template <int RB>  // 32-wide rank blocks (0 = packing only)
__global__ __launch_bounds__(256) void bwd_pack_dy_kernel(BwdPackDyArgs a) {
  constexpr int kRB = RB > 0 ? RB : 1;
  __shared__ float red[4][kRB][16][64];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t mb = blockIdx.x / a.n_slices, sl = blockIdx.x % a.n_slices;
  if (mb >= a.n_row_blocks) return;
  if (a.blk_range && a.blk_range[mb] < 0) return;  // block without rows (grouped calls): never consumed
  const uint32_t i = lane & 31u, h = lane >> 5;
  const uint32_t p = mb * 32u + i;
  int src = -1;
  if (a.src_row) src = a.src_row[p]; else if (p < a.M) src = (int)p;
  if (src >= (int)a.M) src = -1;
  const uint32_t range = (RB > 0 && a.blk_range) ? (uint32_t)a.blk_range[mb] : 0u;
  const uint32_t glo = range & 0xffffu, ghi = range >> 16;
  const uint32_t rowgrp = (RB > 0 && a.slot_group && ghi > glo) ? (uint32_t)a.slot_group[p] : glo;
  const bool vec = (a.N & 7u) == 0;
  v16f acc[kRB];
#pragma unroll
  for (int b = 0; b < kRB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;
  const uint32_t g_end = (sl + 1u) * a.groups_per_slice < a.n_col_groups ? (sl + 1u) * a.groups_per_slice : a.n_col_groups;
  for (uint32_t G = sl * a.groups_per_slice + wave; G < g_end; G += 4u) {
    // piece t = 4 q + 2 ch + part: the 8 columns 128 G + 64 q + 32 ch + 16 h + 8 part .. + 7 of the lane's row
    v8us pc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const uint32_t col = 128u * G + 64u * (t >> 2) + 32u * ((t >> 1) & 1) + 16u * h + 8u * (t & 1);
      if (src >= 0 && vec && col + 8u <= a.N) {
        pc[t] = *reinterpret_cast<const v8us*>(a.dy + (size_t)src * a.N + col);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) pc[t][e] = (src >= 0 && col + e < a.N) ? a.dy[(size_t)src * a.N + col + e] : (uint16_t)0;
      }
    }
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // element e < 4 of packed block j: column 4 e + j of the first 16, e >= 4: of the second 16
        v8us o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[e] = pc[4 * q + ((4 * e + j) >> 3)][(4 * e + j) & 7];
          o[4 + e] = pc[4 * q + 2 + ((4 * e + j) >> 3)][(4 * e + j) & 7];
        }
        const size_t off = ((((size_t)mb * a.NB + 4u * G + j) * 2u + q) * 64u + lane) * 16u;
        *reinterpret_cast<v8us*>(a.dyp + off) = o;
      }
    if constexpr (RB > 0) {
      // a block at a group boundary runs once per group with the other groups' rows zeroed
      for (uint32_t grp = glo; grp <= ghi; ++grp) {
        const bool mine = src >= 0 && rowgrp == grp;
        const uint16_t* bg = a.lora_b + (size_t)grp * a.r * a.N;
        v8us wb[RB][8];
#pragma unroll
        for (int b = 0; b < RB; ++b)
#pragma unroll
          for (int t = 0; t < 8; ++t) {
            const uint32_t col = 128u * G + 64u * (t >> 2) + 32u * ((t >> 1) & 1) + 16u * h + 8u * (t & 1);
            const uint32_t j = b * 32u + i;
            const v8us zero = {0, 0, 0, 0, 0, 0, 0, 0};
            wb[b][t] = (j < a.r && col + 8u <= a.N) ? *reinterpret_cast<const v8us*>(bg + (size_t)j * a.N + col) : zero;
          }
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const v8us zero = {0, 0, 0, 0, 0, 0, 0, 0};
          const v8bf xa = __builtin_bit_cast(v8bf, mine ? pc[t] : zero);
#pragma unroll
          for (int b = 0; b < RB; ++b)
            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa, __builtin_bit_cast(v8bf, wb[b][t]), acc[b], 0, 0, 0);
        }
      }
    }
  }
  if constexpr (RB > 0) {
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) red[wave][b][e][lane] = acc[b][e];
    __syncthreads();
    for (uint32_t q = threadIdx.x; q < RB * 1024u; q += 256u) {
      const uint32_t l = q & 63u, e = (q >> 6) & 15u, b = q >> 10;
      const float sum = ((red[0][b][e][l] + red[1][b][e][l]) + red[2][b][e][l]) + red[3][b][e][l];
      const uint32_t row = 8u * (e >> 2) + 4u * (l >> 5) + (e & 3u), col = b * 32u + (l & 31u);
      a.rpart[((size_t)sl * a.slots + mb * 32u + row) * kBwdRankStride + col] = sum;
    }
  }
}

// r of a 32-row block: the slices' partial sums added in slice order; written raw (for dscaling),
// scaled by the row's group (for dA), and the scaled value split exactly into three bf16 terms in
// the operand order of the pull-back epilogue, rp[block][kk][term][lane][8].
struct BwdRFinishArgs {
  const float* rpart; const int32_t* slot_group; const int32_t* blk_range; const float* lora_scaling;
  float* r_raw; float* rs; unsigned char* rp;
  uint32_t n_slices, slots, nkk, cols;  // cols = 16 * nkk rounded up to 32
};

__global__ __launch_bounds__(256) void bwd_r_finish_kernel(BwdRFinishArgs a) {
  __shared__ float zs[32][kBwdRankStride + 1];
  const uint32_t pb = blockIdx.x;
  if (a.blk_range && a.blk_range[pb] < 0) return;  // block without rows (grouped calls): never consumed
  for (uint32_t q = threadIdx.x; q < 32u * a.cols; q += 256u) {
    const uint32_t row = q / a.cols, col = q % a.cols, slot = pb * 32u + row;
    float raw = 0.0f;
    for (uint32_t sl = 0; sl < a.n_slices; ++sl) raw += a.rpart[((size_t)sl * a.slots + slot) * kBwdRankStride + col];
    a.r_raw[(size_t)slot * kBwdRankStride + col] = raw;
    if (!a.rp) continue;  // plain sum of the slices (the z table)
    const uint32_t gr = a.slot_group ? (uint32_t)a.slot_group[slot] : 0u;
    const float scaled = raw * a.lora_scaling[gr];
    a.rs[(size_t)slot * kBwdRankStride + col] = scaled;
    zs[row][col] = scaled;
  }
  if (!a.rp) return;
  __syncthreads();
  for (uint32_t q = threadIdx.x; q < a.nkk * 3u * 64u; q += 256u) {
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
      o[e] = (unsigned short)(term == 0 ? b0 : (term == 1 ? b1 : b2));
    }
    *reinterpret_cast<v8us*>(a.rp + (((size_t)pb * a.nkk + kk) * 3u + term) * kBlockBytes + l * 16u) = o;
  }
}

// ---------------------------------------------------------------------------------------
// Small per-call tables: LoRA A in B-operand order for the pull-back epilogue,
//   ap[group][k block][kk][64 lanes][8]: lane (c, h) holds A[group][32 kb + c][16 kk + 8 h + 0..7],
// and the per-channel scales in packed column order, swp[p] = sw[packed_to_orig_col(p)].
// ---------------------------------------------------------------------------------------
__device__ inline void lora_a_operand_item(const uint16_t* __restrict__ a, unsigned char* __restrict__ ap,
                                           uint32_t n_groups, uint32_t K, uint32_t r, uint32_t kb32, uint32_t nkk,
                                           uint64_t idx) {
  const uint64_t total = (uint64_t)n_groups * kb32 * nkk * 64u;
  if (idx >= total) return;
  const uint32_t l = (uint32_t)(idx & 63u);
  const uint64_t rest = idx >> 6;
  const uint32_t kk = (uint32_t)(rest % nkk);
  const uint64_t gc = rest / nkk;
  const uint32_t kb = (uint32_t)(gc % kb32), grp = (uint32_t)(gc / kb32);
  const uint32_t k = kb * 32u + (l & 31u);
  v8us o = {0, 0, 0, 0, 0, 0, 0, 0};
  if (k < K) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t row = 16u * kk + 8u * (l >> 5) + e;
      if (row < r) o[e] = a[((size_t)grp * K + k) * r + row];
    }
  }
  *reinterpret_cast<v8us*>(ap + idx * 16u) = o;
}

struct BwdPrepArgs {
  const int32_t* idx;        // adapter per row, or null
  int32_t* src_row; int32_t* dst_pos; int32_t* slot_group; int32_t* blk_range; int32_t* group_off;
  const uint16_t* lora_a;    // bf16 [n_groups, K, r]
  uint16_t* at;              // bf16 [n_groups, r, K]
  unsigned char* ap;
  const float* sw; float* swp;
  uint32_t M, K, N, N_pad, n_groups, r, nkk, kb32, slots, route_blocks, a_blocks, ap_blocks;
};

__global__ __launch_bounds__(1024) void bwd_prep_kernel(BwdPrepArgs p) {
  uint32_t b = blockIdx.x;
  if (b < p.route_blocks) {
    if (p.idx) {
      route_rows_block(p.idx, p.M, p.n_groups, p.slots, p.src_row, p.dst_pos, p.slot_group, p.blk_range, p.group_off, true);
    } else {  // one adapter for every row: identity order, everything in group 0
      for (uint32_t g = threadIdx.x; g <= p.n_groups; g += 1024u) p.group_off[g] = g == 0 ? 0 : (int)p.M;
    }
    return;
  }
  b -= p.route_blocks;
  if (b < p.a_blocks) {
    lora_a_transpose_item(p.lora_a, p.at, p.n_groups, p.K, p.r, (uint64_t)b * 1024u + threadIdx.x);
    return;
  }
  b -= p.a_blocks;
  if (b < p.ap_blocks) {
    lora_a_operand_item(p.lora_a, p.ap, p.n_groups, p.K, p.r, p.kb32, p.nkk, (uint64_t)b * 1024u + threadIdx.x);
    return;
  }
  b -= p.ap_blocks;
  const uint32_t c = b * 1024u + threadIdx.x;
  if (c < p.N_pad) {
    const uint32_t n = packed_to_orig_col(c);
    p.swp[c] = n < p.N ? p.sw[n] : 0.0f;
  }
}

// ---------------------------------------------------------------------------------------
// Tables of a grouped (per-expert) backward: the rows arrive sorted by group, group g owning
// group_sizes[g] consecutive rows, and groups_per_weight consecutive groups share a frozen weight
// (skyrl/tx/layers/lora.py:394-444).  Every weight's rows start at a multiple of the pull-back's tile rows
// (256 slots, or 128 when the weights average few rows), so that
// a pull-back tile never mixes two weights; inside a weight the groups follow each other without
// gaps, exactly as the adapters of a dense call over that weight's rows would.
//   src_row / dst_pos / slot_group / blk_range   as in the dense call; blk_range -1 for 32-slot blocks without a
//                                                row: no kernel prepares or consumes their operands
//   group_beg[g], group_end[g]                   slots of group g
//   tile_weight[t]                               weight of tile t | its rows << 16, -1 beyond the slots in use
//   chunk_tab[c] = (group, first slot, rows)     the 512-row chunks of the LoRA cotangents; rows 0 beyond
//   chunk0[g]                                    first chunk of group g (n_groups + 1 entries)
// One workgroup of 1024 threads.  Rows beyond sum(group_sizes) get no slot; their dx rows are cleared.
// ---------------------------------------------------------------------------------------
struct BwdGroupTables {
  int32_t* src_row; int32_t* dst_pos; int32_t* slot_group; int32_t* blk_range;
  int32_t* group_beg; int32_t* group_end; int32_t* tile_weight; int32_t* chunk_tab; int32_t* chunk0;
};

__device__ inline void route_weight_groups_block(const int32_t* __restrict__ group_sizes, uint32_t M, uint32_t n_groups,
                                                 uint32_t gpw, uint32_t slots, uint32_t max_chunks, BwdGroupTables t,
                                                 uint16_t* __restrict__ dx, uint32_t K, uint32_t tile_rows) {
  const int pad = (int)tile_rows;  // 256, or 128 for the pull-back's 128-row tiles
  __shared__ int row_start[kMaxGroups + 1];
  __shared__ int slot_beg[kMaxGroups + 1];
  __shared__ int slot_end[kMaxGroups];
  __shared__ int chunk_first[kMaxGroups + 1];
  const uint32_t tid = threadIdx.x;
  if (tid < n_groups) row_start[tid] = group_sizes[tid];  // sizes first, starts below
  __syncthreads();
  if (tid == 0) {
    int r = 0, p = 0, ch = 0;
    for (uint32_t g = 0; g < n_groups; ++g) {
      if (g % gpw == 0) p = (p + pad - 1) & ~(pad - 1);
      int sz = row_start[g];
      if (sz < 0) sz = 0;
      if (r + sz > (int)M) sz = (int)M - r;
      row_start[g] = r;
      slot_beg[g] = p;
      chunk_first[g] = ch;
      r += sz;
      p += sz;
      slot_end[g] = p;
      ch += (sz + (int)kBwdChunkRows - 1) / (int)kBwdChunkRows;
    }
    row_start[n_groups] = r;
    slot_beg[n_groups] = p;
    chunk_first[n_groups] = ch;
  }
  for (uint32_t p = tid; p < slots; p += 1024) { t.src_row[p] = -1; t.slot_group[p] = 0; }
  for (uint32_t i = tid; i < M; i += 1024) t.dst_pos[i] = -1;
  for (uint32_t c = tid; c < max_chunks; c += 1024) {
    t.chunk_tab[3u * c] = 0; t.chunk_tab[3u * c + 1u] = 0; t.chunk_tab[3u * c + 2u] = 0;
  }
  __syncthreads();
  for (uint32_t b = tid; b < slots / 32u; b += 1024) t.blk_range[b] = -1;
  for (uint32_t tl = tid; tl < slots / tile_rows; tl += 1024) t.tile_weight[tl] = -1;
  for (uint32_t g = tid; g <= n_groups; g += 1024) t.chunk0[g] = chunk_first[g];
  if (tid < n_groups) { t.group_beg[tid] = slot_beg[tid]; t.group_end[tid] = slot_end[tid]; }
  __syncthreads();
  const uint32_t wave = tid >> 6, lane = tid & 63;
  for (uint32_t g = wave; g < n_groups; g += 16) {
    const int r0 = row_start[g], cnt = row_start[g + 1] - r0, p0 = slot_beg[g];
    for (int i = (int)lane; i < cnt; i += 64) {
      t.src_row[p0 + i] = r0 + i;
      t.dst_pos[r0 + i] = p0 + i;
      t.slot_group[p0 + i] = (int)g;
    }
    const int nch = chunk_first[g + 1] - chunk_first[g];
    for (int c = (int)lane; c < nch; c += 64) {
      const int s0 = p0 + c * (int)kBwdChunkRows;
      const int rows = slot_end[g] - s0 < (int)kBwdChunkRows ? slot_end[g] - s0 : (int)kBwdChunkRows;
      int32_t* e = t.chunk_tab + 3 * (chunk_first[g] + c);
      e[0] = (int)g; e[1] = s0; e[2] = rows;
    }
  }
  // per weight: its tiles, and for every 32-slot block the groups its rows belong to; blocks and
  // padding slots without a row name the weight's last group that has rows (or its first group)
  const uint32_t n_weights = n_groups / gpw;
  for (uint32_t w = wave; w < n_weights; w += 16) {
    const uint32_t g0 = w * gpw, g1 = g0 + gpw;  // groups of this weight
    const int wb = slot_beg[g0], we = slot_end[g1 - 1];
    if (we == wb) continue;  // no rows: no tile
    const int wpad = (we + pad - 1) & ~(pad - 1);
    int glast = (int)g0;
    for (uint32_t g = g0; g < g1; ++g)
      if (slot_end[g] > slot_beg[g]) glast = (int)g;
    for (int tl = wb / pad + (int)lane; tl < wpad / pad; tl += 64) {
      const int rows = we - tl * pad < pad ? we - tl * pad : pad;
      t.tile_weight[tl] = (int)w | (rows << 16);
    }
    for (int p = we + (int)lane; p < wpad; p += 64) t.slot_group[p] = glast;
    for (int b = wb / 32 + (int)lane; b < (we + 31) / 32; b += 64) {  // blocks without a row stay at -1
      const int p0 = b * 32, p1 = p0 + 31 < we ? p0 + 31 : we - 1;
      int lo = glast, hi = glast;
      for (uint32_t g = g0; g < g1; ++g) {
        if (p0 >= slot_beg[g] && p0 < slot_end[g]) lo = (int)g;
        if (p1 >= slot_beg[g] && p1 < slot_end[g]) hi = (int)g;
      }
      t.blk_range[b] = lo | (hi << 16);
    }
  }
  if (dx) {
    const size_t begin = (size_t)row_start[n_groups] * K, end = (size_t)M * K;
    for (size_t i = begin + tid; i < end; i += 1024) dx[i] = 0;
  }
}

struct BwdGroupedPrepArgs {
  const int32_t* group_sizes;
  BwdGroupTables tab;
  const uint16_t* lora_a;    // bf16 [n_groups, K, r]
  uint16_t* at;              // bf16 [n_groups, r, K]
  unsigned char* ap;
  const float* sw;           // f32 [n_weights, N]
  float* swp;                // f32 [n_weights][sw_stride] in packed column order
  uint16_t* dx;              // rows beyond the groups are cleared
  uint32_t M, K, N, N_pad, n_groups, gpw, n_weights, r, nkk, kb32, slots, max_chunks, sw_stride;
  uint32_t a_blocks, ap_blocks, sw_blocks_per_weight;
  uint32_t tile_rows;        // slots every weight's rows are padded to: 256 or 128
};

__global__ __launch_bounds__(1024) void bwd_grouped_prep_kernel(BwdGroupedPrepArgs p) {
  uint32_t b = blockIdx.x;
  if (b == 0) {
    route_weight_groups_block(p.group_sizes, p.M, p.n_groups, p.gpw, p.slots, p.max_chunks, p.tab, p.dx, p.K, p.tile_rows);
    return;
  }
  b -= 1u;
  if (b < p.a_blocks) {
    lora_a_transpose_item(p.lora_a, p.at, p.n_groups, p.K, p.r, (uint64_t)b * 1024u + threadIdx.x);
    return;
  }
  b -= p.a_blocks;
  if (b < p.ap_blocks) {
    lora_a_operand_item(p.lora_a, p.ap, p.n_groups, p.K, p.r, p.kb32, p.nkk, (uint64_t)b * 1024u + threadIdx.x);
    return;
  }
  b -= p.ap_blocks;
  const uint32_t w = b / p.sw_blocks_per_weight, c = (b % p.sw_blocks_per_weight) * 1024u + threadIdx.x;
  if (w < p.n_weights && c < p.N_pad) {
    const uint32_t n = packed_to_orig_col(c);
    p.swp[(size_t)w * p.sw_stride + c] = n < p.N ? p.sw[(size_t)w * p.N + n] : 0.0f;
  }
}

// ---------------------------------------------------------------------------------------
// dx = dyp @ bf16(W * sw).T (+ rs @ A.T), one bf16 cast.
// Workgroup = 8 waves (2 along rows x 4 along k), tile 256 rows x 256 k, wave tile 128 x 64
// (4 x 2 accumulator blocks of v_mfma_f32_32x32x16_bf16).  The contraction runs over n in stages
// of one 32-wide n block.  A stage's dy panel (16 KiB), weight blocks (8 KiB) and scales travel
// HBM/L2 -> LDS with direct-to-LDS loads five stages ahead.  While the matrix core works on stage
// nb, the vector ALU prepares the weight operands of stage nb + 1: each wave transposes its two
// blocks with the identity MFMA, scales, rounds to bf16 and keeps them in registers.
// ---------------------------------------------------------------------------------------
constexpr int kBwdStages = 6;
constexpr int kBwdAhead = kBwdStages - 1;  // stages between a load and its use
constexpr int kBwdStagePanel = 16384;      // dy: 8 row blocks x 2 halves
constexpr int kBwdStageWeight = 8192;      // 8 k blocks of the n block
constexpr int kBwdStageBytes = kBwdStagePanel + kBwdStageWeight + 1024;  // + a 1 KiB chunk of scales (the stage's 32 lead it)
constexpr int kBwdLdsBytes = kBwdStages * kBwdStageBytes;
constexpr int kBwdLoadsPerStage = 4;  // direct-to-LDS loads per wave per stage: 2 panel chunks, 1 weight block, scales
constexpr int kBwdScalePad = 256;     // floats readable past the last stage's scales

struct BwdDxArgs {
  const unsigned char* dyp;   // packed dy
  const unsigned char* wp;    // packed weight
  const float* swp;           // scales in packed column order [N_pad + 32]
  const unsigned char* rp;    // packed rs fragments [slots/32][NKK][3][64][8] or null
  const unsigned char* ap;    // packed A operands or null
  const int32_t* src_row; const int32_t* slot_group; const int32_t* blk_range;
  uint16_t* dx;               // bf16 [M, K]
  uint32_t M, K, KB, NB, tiles_m, tiles_k;
  // grouped calls: weight | rows << 16 of every 256-slot tile (-1: tile without rows; the rows fill the
  // tile from its first slot), the bytes between two packed weights and the floats between two scale
  // tables; null / 0 for one weight
  const int32_t* tile_weight;
  size_t w_stride;
  uint32_t sw_stride;
};

// ROWS128: the tile is 128 rows x 512 k (the eight waves side by side along k, the same 128 x 64 wave
// tile): a stage then holds half the dy panel and twice the weight blocks, the same bytes and the same
// four loads per wave.  For grouped calls whose weights own few rows each: half the padding per weight,
// and every wave has rows.
template <int NKK, bool ROWS128 = false>
__global__ __launch_bounds__(512, 1) void bwd_dx_kernel(BwdDxArgs g) {
  constexpr int kRowBlocks = ROWS128 ? 4 : 8, kKBlocks = ROWS128 ? 16 : 8;  // of a tile
  constexpr int kPanel = kRowBlocks * 2048, kWeight = kKBlocks * kBlockBytes;
  static_assert(kPanel + kWeight + 1024 == kBwdStageBytes, "a stage keeps its size in both geometries");
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wrow = ROWS128 ? 0 : wave >> 2, wcol = ROWS128 ? wave : wave & 3;
  const int c = lane & 31, h = lane >> 5;
  const int NBi = (int)g.NB;  // a multiple of 8

  // identity operand of the transposing MFMA: lane (column c, k half h) holds byte 1 at k == c
  v4i ident = {0, 0, 0, 0};
  {
    const int word = ((c >> 4) == h) ? (int)(1u << (8 * (c & 3))) : 0;
    const int wi = (c & 15) >> 2;
    ident[0] = wi == 0 ? word : 0; ident[1] = wi == 1 ? word : 0;
    ident[2] = wi == 2 ? word : 0; ident[3] = wi == 3 ? word : 0;
  }

  const uint32_t ntile = g.tiles_m * g.tiles_k;
  const uint32_t wgs_per_xcd = gridDim.x >> 3, xcd = blockIdx.x & 7u;
  // band-major tile order: 4 row tiles x all k tiles, so an XCD's workgroups share panels.  One weight:
  // every XCD walks a contiguous range of bands.  Grouped calls: the bands are dealt round-robin to the
  // XCDs, because the slots in use end before the last bands and a contiguous split would leave the
  // last XCDs without work.
  const uint32_t band_tiles = 4u * g.tiles_k, n_bands = (g.tiles_m + 3u) / 4u;
  const uint32_t per_xcd = g.tile_weight ? ((n_bands + 7u) / 8u) * band_tiles : (ntile + 7u) / 8u;
  for (uint32_t ti = blockIdx.x >> 3; ti < per_xcd; ti += wgs_per_xcd) {
    uint32_t band, in_band;
    if (g.tile_weight) {
      band = xcd + 8u * (ti / band_tiles);
      in_band = ti % band_tiles;
      if (band >= n_bands) break;
    } else {
      const uint32_t t = xcd * per_xcd + ti;
      if (t >= ntile) break;
      band = t / band_tiles;
      in_band = t - band * band_tiles;
    }
    const uint32_t band_rows = (g.tiles_m - band * 4u) < 4u ? (g.tiles_m - band * 4u) : 4u;
    if (in_band >= band_rows * g.tiles_k) continue;  // a last band with fewer than 4 row tiles (grouped order only)
    const uint32_t tm = band * 4u + in_band % band_rows, tk = in_band / band_rows;
    int tw = 0;
    int n_act = 4;  // 32-row blocks of this wave that hold rows: the others skip their matrix-core work
    // row block whose dy panel this wave fetches: both 1 KiB halves, or one half of it in a 128-row tile
    uint32_t load_rb = ROWS128 ? (uint32_t)wave >> 1 : (uint32_t)wave;
    if (g.tile_weight) {
      const int tv = g.tile_weight[tm];
      if (tv < 0) continue;  // workgroup-uniform: no row lives in this tile
      tw = tv & 0xffff;
      const int live_blocks = ((tv >> 16) + 31) / 32;
      const int live = live_blocks - wrow * 4;
      n_act = live < 0 ? 0 : (live > 4 ? 4 : live);
      // a block without rows is never multiplied: its slot is filled from block 0 of the tile, which
      // is in the caches anyway, instead of streaming unused memory (the load count stays the same)
      if ((int)load_rb >= live_blocks) load_rb = 0u;
    }
    n_act = __builtin_amdgcn_readfirstlane(n_act);
    const float* swp_t = g.swp + (size_t)tw * g.sw_stride;

    // this wave's two panel chunks of a stage (row block = wave, halves q = 0, 1) and its weight block
    const unsigned char* Ag = g.dyp + ((size_t)(tm * (uint32_t)kRowBlocks + load_rb) * g.NB) * 2048u +
                              (ROWS128 ? (wave & 1) * 1024 : 0) + lane * 16;
    const uint32_t kbw = tk * (uint32_t)kKBlocks + (uint32_t)wcol * 2u;  // first of the two k blocks this wave multiplies
    // the block(s) it loads: one of eight, or its own two of sixteen; blocks past the weight repeat the last
    const uint32_t kbl0 = tk * (uint32_t)kKBlocks + (ROWS128 ? 2u * (uint32_t)wave : (uint32_t)wave);
    const uint32_t kbl = kbl0 < g.KB ? kbl0 : g.KB - 1u;
    const uint32_t kbl1 = kbl0 + 1u < g.KB ? kbl0 + 1u : g.KB - 1u;
    const unsigned char* Bg = g.wp + (size_t)tw * g.w_stride + (size_t)kbl * kBlockBytes + lane * 16;
    const unsigned char* Bg1 = g.wp + (size_t)tw * g.w_stride + (size_t)kbl1 * kBlockBytes + lane * 16;
    const size_t nb_stride = (size_t)g.KB * kBlockBytes;

    auto issue = [&](int nb) {
      unsigned char* St = lds + (nb % kBwdStages) * kBwdStageBytes;
      const unsigned char* src = Ag + (size_t)nb * 2048u;
      if constexpr (ROWS128) {
        load_1k_to_lds(src, St + wave * kBlockBytes);
        load_1k_to_lds(Bg + (size_t)nb * nb_stride, St + kPanel + (wave * 2) * kBlockBytes);
        load_1k_to_lds(Bg1 + (size_t)nb * nb_stride, St + kPanel + (wave * 2 + 1) * kBlockBytes);
      } else {
        load_1k_to_lds(src, St + (wave * 2) * kBlockBytes);
        load_1k_to_lds(src + 1024, St + (wave * 2 + 1) * kBlockBytes);
        load_1k_to_lds(Bg + (size_t)nb * nb_stride, St + kPanel + wave * kBlockBytes);
      }
      // every wave fetches the same 1 KiB of scales (the stage's 32 lead it) to the same place
      load_1k_to_lds(reinterpret_cast<const unsigned char*>(swp_t + 32 * nb) + lane * 16, St + kPanel + kWeight);
    };

    v16f acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto transpose_block = [&](const v4i& rawb) -> v16i {
      v16i z16;
#pragma unroll
      for (int e = 0; e < 16; ++e) z16[e] = 0;
      return __builtin_amdgcn_mfma_i32_32x32x32_i8(rawb, ident, z16, 0, 0, 0);
    };
    // rows 8 gq + 4 h + 0..3 of a transposed block: bf16(float(code) * scale), the per-element
    // weight of the reference's pull-back
    auto convert4 = [&](const v16i& tr, const v4f& s4, int gq, uint32_t (&pk)[8]) {
      const float f0 = (float)tr[4 * gq + 0] * s4[0], f1 = (float)tr[4 * gq + 1] * s4[1];
      const float f2 = (float)tr[4 * gq + 2] * s4[2], f3 = (float)tr[4 * gq + 3] * s4[3];
      pk[2 * gq] = pack_bf16x2(f0, f1);
      pk[2 * gq + 1] = pack_bf16x2(f2, f3);
    };
    auto to_operands = [&](const uint32_t (&pk)[8], v8bf (&bq)[2]) {
      bq[0] = __builtin_bit_cast(v8bf, v4i{(int)pk[0], (int)pk[1], (int)pk[2], (int)pk[3]});
      bq[1] = __builtin_bit_cast(v8bf, v4i{(int)pk[4], (int)pk[5], (int)pk[6], (int)pk[7]});
    };
    auto panel_frag = [&](int nb, int pair) -> v8bf {  // pair = 4 q + row block
      const unsigned char* St = lds + (nb % kBwdStages) * kBwdStageBytes;
      return __builtin_bit_cast(
          v8bf, *reinterpret_cast<const v4i*>(St + ((wrow * 4 + (pair & 3)) * 2 + (pair >> 2)) * kBlockBytes + lane * 16));
    };
    // The weight blocks and scales of the next stage are read from LDS with explicit instructions:
    // a compiler-visible read of memory that direct-to-LDS loads write makes the compiler drain
    // every outstanding load first (it cannot tell the stages apart), which would serialize the
    // pipeline.  The six values are valid after next_wait().
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)lds;
    struct NextRegs { v4i raw[2]; v4f s4[4]; };
    auto next_read = [&](int nb1, NextRegs& r) {
      const uint32_t st = lds_base + (nb1 % kBwdStages) * kBwdStageBytes + kPanel;
      const uint32_t wa = st + (wcol * 2) * kBlockBytes + lane * 16;
      const uint32_t sa = st + kWeight + 16 * h;
      asm volatile("ds_read_b128 %0, %6\n\tds_read_b128 %1, %6 offset:1024\n\t"
                   "ds_read_b128 %2, %7\n\tds_read_b128 %3, %7 offset:32\n\t"
                   "ds_read_b128 %4, %7 offset:64\n\tds_read_b128 %5, %7 offset:96"
                   : "=&v"(r.raw[0]), "=&v"(r.raw[1]), "=&v"(r.s4[0]), "=&v"(r.s4[1]), "=&v"(r.s4[2]), "=&v"(r.s4[3])
                   : "v"(wa), "v"(sa)
                   : "memory");
    };
    auto next_wait = [&](NextRegs& r) {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(r.raw[0]), "+v"(r.raw[1]), "+v"(r.s4[0]), "+v"(r.s4[1]), "+v"(r.s4[2]), "+v"(r.s4[3])
                   :
                   : "memory");
    };

    // One stage: 16 MFMAs of stage nb against the dy panel in LDS; between them the operands of
    // stage nb + 1 are prepared (vector ALU work under the matrix core's shadow).
    auto stage = [&](int nb, const v8bf (&bqC)[2][2], v8bf (&bqN)[2][2], bool convert_next) {
      if (n_act == 0) return;  // wave-uniform: a wave without rows only feeds the pipeline
      NextRegs nx;
      v16i tr;
      uint32_t pk[8];
      if (convert_next) next_read(nb + 1, nx);
      v8bf af = panel_frag(nb, 0);
#pragma unroll
      for (int pair = 0; pair < 8; ++pair) {
        const int q = pair >> 2, rb = pair & 3;
        v8bf af_next = af;
        if (pair < 7) af_next = panel_frag(nb, pair + 1);
        if (rb < n_act) {
          acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bqC[0][q], acc[rb][0], 0, 0, 0);
          acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bqC[1][q], acc[rb][1], 0, 0, 0);
        }
        if (convert_next) {
          if (pair == 0) {
            next_wait(nx);
            tr = transpose_block(nx.raw[0]);
          } else {
            const int cstep = pair - 1;  // conversion step: k block cstep / 4, rows 8 (cstep % 4) + ...
            convert4(tr, nx.s4[cstep & 3], cstep & 3, pk);
            if (cstep == 3) {
              to_operands(pk, bqN[0]);
              tr = transpose_block(nx.raw[1]);
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        af = af_next;
      }
      if (convert_next) {
        convert4(tr, nx.s4[3], 3, pk);
        to_operands(pk, bqN[1]);
      }
    };

    // ---- main loop.  Stage nb issues the loads of stage nb + 5.
    v8bf bqA[2][2], bqB[2][2];
    wait_vmcnt<0>();  // stores of the previous tile
    lds_barrier();
#pragma unroll
    for (int i = 0; i < kBwdAhead; ++i) issue(i);  // NB >= 8
    wait_vmcnt<0>();
    lds_barrier();
    if (n_act > 0) {  // operands of stage 0
      NextRegs nx;
      next_read(0, nx);
      next_wait(nx);
      uint32_t pk[8];
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        const v16i tr = transpose_block(nx.raw[cb]);
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) convert4(tr, nx.s4[gq], gq, pk);
        to_operands(pk, bqA[cb]);
      }
    }
    const int NB_main = NBi - kBwdAhead;  // stages that still have loads to issue; odd
    int nb = 0;
    for (; nb + 1 < NB_main; nb += 2) {
      // stage nb + 1 (and so stage nb) is older than the loads of the last three stages
      wait_vmcnt<(kBwdAhead - 2) * kBwdLoadsPerStage>();
      lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
      issue(nb + kBwdAhead);
      stage(nb, bqA, bqB, true);
      __builtin_amdgcn_sched_barrier(0);
      wait_vmcnt<(kBwdAhead - 2) * kBwdLoadsPerStage>();
      lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
      issue(nb + 1 + kBwdAhead);
      stage(nb + 1, bqB, bqA, true);
      __builtin_amdgcn_sched_barrier(0);
    }
    for (; nb < NBi; nb += 2) {  // drain: fewer loads in flight than the count above assumes
      wait_vmcnt<0>();
      lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
      if (nb + kBwdAhead < NBi) issue(nb + kBwdAhead);
      stage(nb, bqA, bqB, true);
      __builtin_amdgcn_sched_barrier(0);
      wait_vmcnt<0>();
      lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
      if (nb + 1 + kBwdAhead < NBi) issue(nb + 1 + kBwdAhead);
      stage(nb + 1, bqB, bqA, nb + 2 < NBi);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue: + rs @ A.T, one cast, rows back to their original positions
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const uint32_t pbase = tm * (uint32_t)(kRowBlocks * 32) + (uint32_t)wrow * 128u + rb * 32u;
      const uint32_t blk = pbase / 32u;
      const int src_lane = g.src_row ? g.src_row[pbase + c] : (int)(pbase + c);
      const bool row_ok = src_lane >= 0 && src_lane < (int)g.M;
      const uint32_t off_lane = row_ok ? (uint32_t)src_lane * g.K : 0xffffffffu;
      if (__builtin_amdgcn_ballot_w64(row_ok) == 0) continue;  // wave-uniform: no row of this block exists
      const uint32_t range = (NKK > 0 && g.blk_range) ? (uint32_t)g.blk_range[blk] : 0u;
      const int glo = (int)(range & 0xffffu), ghi = (int)(range >> 16);
      const int grp_lane = (NKK > 0 && g.slot_group && ghi > glo) ? g.slot_group[pbase + c] : glo;
      const int row_addr = 16 * h;
      for (int gi = glo; gi <= ghi; ++gi) {  // a block at a group boundary runs once per group
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
          const uint32_t kb = kbw + cb;
          if (kb >= g.KB) continue;  // wave-uniform
          const uint32_t kcol = kb * 32u + c;
          v16f y = acc[rb][cb];
          if constexpr (NKK > 0) {
            const unsigned char* rb0 = g.rp + (size_t)blk * NKK * 3u * kBlockBytes + lane * 16;
            const unsigned char* ab0 = g.ap + ((size_t)gi * g.KB + kb) * NKK * kBlockBytes + lane * 16;
            v16f low;
#pragma unroll
            for (int e = 0; e < 16; ++e) low[e] = 0.0f;
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk) {
              const v8bf ab = __builtin_bit_cast(v8bf, *reinterpret_cast<const v8us*>(ab0 + kk * kBlockBytes));
#pragma unroll
              for (int t3 = 2; t3 >= 0; --t3) {
                const v8bf rf = __builtin_bit_cast(v8bf, *reinterpret_cast<const v8us*>(rb0 + (kk * 3 + t3) * kBlockBytes));
                low = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rf, ab, low, 0, 0, 0);
              }
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) y[e] = y[e] + low[e];
          }
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int src_lane_addr = row_addr + 4 * (8 * (v >> 2) + (v & 3));
            const uint32_t rowoff = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane_addr, (int)off_lane);
            // every lane takes part in the cross-lane reads: a lane that is switched off (a column
            // beyond K) would hand zeros to the lanes that read from it
            int row_grp = gi;
            if (NKK > 0 && ghi > glo) row_grp = __builtin_amdgcn_ds_bpermute(src_lane_addr, grp_lane);
            const bool ok = (rowoff != 0xffffffffu) & (kcol < g.K) & (row_grp == gi);
            if (ok) g.dx[(size_t)rowoff + kcol] = (uint16_t)f32_to_bf16_bits(y[v]);
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// LoRA cotangents.  Rows are in grouped order; group g owns slots group_off[g] .. group_off[g+1].
// Every group is cut into chunks of 512 rows; chunk c of the call computes, for its rows,
//   partA[c][j][k] = sum_m rs[m][j] * x[m][k]        partB[c][j][n] = sum_m z[m][j] * dy[m][n]
// with float32 accumulation, and a second kernel adds a
// group's chunks in chunk order, scales dB, casts and writes dA [g][K][r], dB [g][r][N], plus
// ds[g] = sum_m sum_j r[m][j] * z[m][j] with r the unscaled dy @ B.T.  Fixed orders: results are
// deterministic.
// ---------------------------------------------------------------------------------------

struct BwdDloraArgs {
  const uint16_t* x;        // bf16 [M, K]
  const uint16_t* dy;       // bf16 [M, N]
  const float* rs;          // f32 [slots][64]  (dy @ B.T) * s
  const float* z;           // f32 [slots][64]  x @ A
  const int32_t* src_row;   // or null
  const int32_t* group_off; // [n_groups + 1]
  const int32_t* chunk_tab; // grouped calls: (group, first slot, rows) per chunk instead of group_off
  float* partA;             // [max_chunks][R][K]
  float* partB;             // [max_chunks][R][N]
  uint32_t M, K, N, n_groups, max_chunks, col_tiles_a, col_tiles_b;
};

// chunk id -> (group, first slot, rows); false beyond the last chunk
__device__ inline bool bwd_find_chunk(const int32_t* group_off, uint32_t n_groups, uint32_t cid, uint32_t& grp,
                                      uint32_t& slot0, uint32_t& rows) {
  uint32_t run = 0;
  for (uint32_t gq = 0; gq < n_groups; ++gq) {
    const uint32_t o0 = (uint32_t)group_off[gq], o1 = (uint32_t)group_off[gq + 1];
    const uint32_t nch = (o1 - o0 + kBwdChunkRows - 1u) / kBwdChunkRows;
    if (cid < run + nch) {
      grp = gq;
      slot0 = o0 + (cid - run) * kBwdChunkRows;
      rows = o1 - slot0 < kBwdChunkRows ? o1 - slot0 : kBwdChunkRows;
      return true;
    }
    run += nch;
  }
  return false;
}

// Matrix-core version.  out[j][c] = sum_m P[m][j] * Q[m][c] contracts over rows, so both operands
// need the row index inside a lane.  P (float32, 32 or 64 rank columns) is split exactly into three
// bf16 terms and staged in LDS in A-operand order.  Q (bf16 rows of x or dy) is read as ordinary
// row fragments and transposed by the matrix core: two v_mfma_f32_32x32x16_bf16 against identity
// halves return Q[m][c] with lane = c and sixteen rows per lane (exact: the values are bf16), which
// packs into the B operands of the contraction over m.  A wave owns 64 columns (two 32-column
// strips) and walks the chunk's 32-row blocks, eight per staging pass of P; a workgroup of four
// waves owns 256 columns.
template <int RB>  // 32-wide rank blocks
__global__ __launch_bounds__(256) void bwd_dlora_kernel(BwdDloraArgs a) {
  // P operands: [row block 8][rank block RB][q 2][term 3][64 lanes][8 bf16]
  extern __shared__ __attribute__((aligned(1024))) unsigned char pop[];
  __shared__ int rowsrc[kBwdStageRows];
  __shared__ uint32_t info[3];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t per_chunk = a.col_tiles_a + a.col_tiles_b;
  const uint32_t cid = blockIdx.x / per_chunk, ct = blockIdx.x % per_chunk;
  if (tid == 0) {
    uint32_t grp = 0, slot0 = 0, rows = 0;
    if (a.chunk_tab) {
      grp = (uint32_t)a.chunk_tab[3u * cid]; slot0 = (uint32_t)a.chunk_tab[3u * cid + 1u];
      rows = (uint32_t)a.chunk_tab[3u * cid + 2u];
    } else if (!bwd_find_chunk(a.group_off, a.n_groups, cid, grp, slot0, rows)) {
      rows = 0;
    }
    info[0] = grp; info[1] = slot0; info[2] = rows;
  }
  __syncthreads();
  const uint32_t slot0 = info[1], rows = info[2];
  if (rows == 0) return;  // workgroup-uniform
  const bool job_a = ct < a.col_tiles_a;
  const float* psrc = job_a ? a.rs : a.z;
  const uint16_t* Q = job_a ? a.x : a.dy;
  const uint32_t C = job_a ? a.K : a.N;
  float* part = job_a ? a.partA : a.partB;
  const uint32_t c = lane & 31u, h = lane >> 5;
  const uint32_t col0 = ((job_a ? ct : ct - a.col_tiles_a) * 4u + wave) * 64u;  // first column of the wave
  const bool active = col0 < C;
  // identity halves: lane (column c, half h) element e is 1 where the contraction slot 8 h + e is column c
  v8us id0 = {0, 0, 0, 0, 0, 0, 0, 0}, id1 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    id0[e] = (c == 8u * h + e) ? (unsigned short)0x3f80 : (unsigned short)0;
    id1[e] = (c == 16u + 8u * h + e) ? (unsigned short)0x3f80 : (unsigned short)0;
  }
  v16f acc[2][RB];
#pragma unroll
  for (int st = 0; st < 2; ++st)
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[st][b][e] = 0.0f;
  const v8us zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  auto load_q = [&](uint32_t bi, v8us (&dst)[2][2]) {  // [strip][column half]: row c of the block, 8 columns
    const int srow = rowsrc[bi * 32u + c];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int hc = 0; hc < 2; ++hc) {
        const uint32_t col = col0 + 32u * st + 16u * hc + 8u * h;
        dst[st][hc] = (srow >= 0 && col + 8u <= C) ? *reinterpret_cast<const v8us*>(Q + (size_t)srow * C + col) : zero8;
      }
  };
  for (uint32_t base = 0; base < rows; base += kBwdStageRows) {
    const uint32_t cnt = rows - base < kBwdStageRows ? rows - base : kBwdStageRows;
    const uint32_t n_blocks = (cnt + 31u) / 32u;
    __syncthreads();  // the previous pass's operands are no longer read
    // stage P: item = (row block, rank block, q, lane); element e is row 16 q + 8 (e / 4) + 4 h + e % 4
    for (uint32_t it = tid; it < n_blocks * RB * 2u * 64u; it += 256u) {
      const uint32_t l = it & 63u, q = (it >> 6) & 1u, jb = (it >> 7) % RB, bi = (it >> 7) / RB;
      const uint32_t j = jb * 32u + (l & 31u), hh = l >> 5;
      v8us t0, t1, t2;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t m = bi * 32u + 16u * q + 8u * (e >> 2) + 4u * hh + (e & 3);
        const float v = m < cnt ? psrc[(size_t)(slot0 + base + m) * kBwdRankStride + j] : 0.0f;
        const uint32_t b0 = f32_to_bf16_bits(v);
        const float r1 = v - bf16_bits_to_f32(b0);
        const uint32_t b1 = f32_to_bf16_bits(r1);
        const float r2 = r1 - bf16_bits_to_f32(b1);
        t0[e] = (unsigned short)b0; t1[e] = (unsigned short)b1; t2[e] = (unsigned short)f32_to_bf16_bits(r2);
      }
      unsigned char* dst = pop + ((((size_t)bi * RB + jb) * 2u + q) * 3u) * kBlockBytes + l * 16u;
      *reinterpret_cast<v8us*>(dst) = t0;
      *reinterpret_cast<v8us*>(dst + kBlockBytes) = t1;
      *reinterpret_cast<v8us*>(dst + 2 * kBlockBytes) = t2;
    }
    for (uint32_t i = tid; i < kBwdStageRows; i += 256u)
      rowsrc[i] = i < cnt ? (a.src_row ? a.src_row[slot0 + base + i] : (int)(slot0 + base + i)) : -1;
    __syncthreads();
    if (!active) continue;
    v8us qf[2][2];
    load_q(0, qf);
    for (uint32_t bi = 0; bi < n_blocks; ++bi) {
      v8us qn[2][2];
      if (bi + 1u < n_blocks) load_q(bi + 1u, qn);
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        v16f tr;
#pragma unroll
        for (int e = 0; e < 16; ++e) tr[e] = 0.0f;
        tr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, qf[st][0]), __builtin_bit_cast(v8bf, id0), tr, 0, 0, 0);
        tr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, qf[st][1]), __builtin_bit_cast(v8bf, id1), tr, 0, 0, 0);
        v4i bq[2];
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) bq[q][e] = (int)pack_bf16x2(tr[8 * q + 2 * e], tr[8 * q + 2 * e + 1]);
#pragma unroll
        for (int b = 0; b < RB; ++b)
#pragma unroll
          for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int t3 = 2; t3 >= 0; --t3) {
              const v8bf pf = __builtin_bit_cast(
                  v8bf, *reinterpret_cast<const v8us*>(pop + ((((size_t)bi * RB + b) * 2u + q) * 3u + t3) * kBlockBytes + lane * 16u));
              acc[st][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf, __builtin_bit_cast(v8bf, bq[q]), acc[st][b], 0, 0, 0);
            }
      }
      if (bi + 1u < n_blocks) {
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int hc = 0; hc < 2; ++hc) qf[st][hc] = qn[st][hc];
      }
    }
  }
  if (!active) return;
  // lane (c, h) holds column col0 + 32 st + c, rank rows 32 b + 8 (v / 4) + 4 h + v % 4
#pragma unroll
  for (int st = 0; st < 2; ++st) {
    const uint32_t col = col0 + 32u * st + c;
    if (col >= C) continue;
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const uint32_t j = b * 32u + 8u * (v >> 2) + 4u * h + (v & 3);
        part[((size_t)cid * (RB * 32u) + j) * C + col] = acc[st][b][v];
      }
  }
}

struct BwdReduceArgs {
  const float* partA; const float* partB;
  const float* r_raw;       // f32 [slots][64] unscaled dy @ B.T
  const float* z;           // f32 [slots][64]
  const float* lora_scaling;
  const int32_t* group_off;
  // grouped calls: first chunk of every group (n_groups + 1) and the groups' slot ranges, in memory
  const int32_t* chunk0_tab; const int32_t* group_beg; const int32_t* group_end;
  uint16_t* d_a;            // bf16 [n_groups, K, r] or null
  uint16_t* d_b;            // bf16 [n_groups, r, N] or null
  float* d_s;               // f32 [n_groups] or null
  uint32_t K, N, r, R, n_groups, blocks_a, blocks_b;
};

__global__ __launch_bounds__(256) void bwd_dlora_reduce_kernel(BwdReduceArgs a) {
  __shared__ uint32_t chunk0_lds[kMaxAdapters + 1];
  __shared__ double red[256];
  const uint32_t tid = threadIdx.x;
  if (!a.chunk0_tab && tid < 64u) {
    // first chunk of every group: the dense tables hold at most 64 groups, so one wave loads all the
    // offsets at once and scans the chunk counts (a serial loop over dependent loads in front of every
    // workgroup of this short kernel cost more than the reduction itself)
    static_assert(kMaxAdapters <= 64, "one wave scans the groups");
    uint32_t cnt = 0;
    if (tid < a.n_groups)
      cnt = ((uint32_t)(a.group_off[tid + 1] - a.group_off[tid]) + kBwdChunkRows - 1u) / kBwdChunkRows;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const uint32_t up = (uint32_t)__shfl_up((int)cnt, o, 64);
      if ((int)tid >= o) cnt += up;
    }
    if (tid < a.n_groups) chunk0_lds[tid + 1u] = cnt;  // inclusive sums
    if (tid == 0) chunk0_lds[0] = 0u;
  }
  __syncthreads();
  auto chunk0 = [&](uint32_t gq) -> uint32_t { return a.chunk0_tab ? (uint32_t)a.chunk0_tab[gq] : chunk0_lds[gq]; };
  auto reduce_ds = [&](uint32_t b) {  // one block per group
    const uint32_t o0 = (uint32_t)(a.group_beg ? a.group_beg[b] : a.group_off[b]);
    const uint32_t o1 = (uint32_t)(a.group_end ? a.group_end[b] : a.group_off[b + 1]);
    // thread = (rank column j, one of four rows per pass); eight passes of loads are in flight at a time:
    // one load pair per iteration left this single workgroup per group waiting out a memory latency per
    // four rows, longer than the rest of the launch takes
    double sum = 0.0;
    const uint32_t j = tid & 63u;
    if (j < a.r) {
      uint32_t slot = o0 + (tid >> 6);
      for (; slot + 28u < o1; slot += 32u) {
        float rv[8], zv[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
          const size_t off = (size_t)(slot + 4u * u) * kBwdRankStride + j;
          rv[u] = a.r_raw[off];
          zv[u] = a.z[off];
        }
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) sum += (double)rv[u] * (double)zv[u];
      }
      for (; slot < o1; slot += 4u) {
        const size_t off = (size_t)slot * kBwdRankStride + j;
        sum += (double)a.r_raw[off] * (double)a.z[off];
      }
    }
    red[tid] = sum;
    __syncthreads();
    for (uint32_t o = 128; o > 0; o >>= 1) {
      if (tid < o) red[tid] += red[tid + o];
      __syncthreads();
    }
    if (tid == 0) a.d_s[b] = (float)red[0];
  };
  // The blocks of ds come first in the grid: each walks all rows of its group and takes longest, so it
  // starts at once and runs beside the short dA / dB blocks instead of after them.
  const uint32_t blocks_s = a.d_s ? a.n_groups : 0u;
  if (blockIdx.x < blocks_s) {
    reduce_ds(blockIdx.x);
    return;
  }
  uint32_t b = blockIdx.x - blocks_s;
  if (b < a.blocks_a) {
    // dA [group][k][j]: a thread per output element, j fastest, so that the stores are contiguous
    const uint64_t e = (uint64_t)b * 256u + tid;
    if (e >= (uint64_t)a.n_groups * a.K * a.r || !a.d_a) return;
    const uint32_t j = (uint32_t)(e % a.r), col = (uint32_t)((e / a.r) % a.K), grp = (uint32_t)(e / ((uint64_t)a.r * a.K));
    float sum = 0.0f;
    for (uint32_t ch = chunk0(grp), ce = chunk0(grp + 1u); ch < ce; ++ch) sum += a.partA[((size_t)ch * a.R + j) * a.K + col];
    a.d_a[e] = (uint16_t)f32_to_bf16_bits(sum);
    return;
  }
  if (b < a.blocks_a + a.blocks_b) {
    // dB [group][j][n]: a thread per four adjacent columns (N is a multiple of 8)
    const uint64_t e = ((uint64_t)(b - a.blocks_a) * 256u + tid) * 4u;
    if (e >= (uint64_t)a.n_groups * a.r * a.N || !a.d_b) return;
    const uint32_t col = (uint32_t)(e % a.N), j = (uint32_t)((e / a.N) % a.r), grp = (uint32_t)(e / ((uint64_t)a.N * a.r));
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t ch = chunk0(grp), ce = chunk0(grp + 1u); ch < ce; ++ch) {
      const float4 v = *reinterpret_cast<const float4*>(a.partB + ((size_t)ch * a.R + j) * a.N + col);
      sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    const float sc = a.lora_scaling[grp];
    *reinterpret_cast<uint2*>(a.d_b + e) = make_uint2(pack_bf16x2(sum.x * sc, sum.y * sc), pack_bf16x2(sum.z * sc, sum.w * sc));
    return;
  }
}

}  // namespace w8a8
