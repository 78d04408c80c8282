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
// One wave per (row block, 128-column group, q): a lane reads 2 x 16 consecutive original columns
// of its row and owns the four packed blocks (j = column % 4) that interleave them.
// ---------------------------------------------------------------------------------------
struct BwdPackDyArgs {
  const uint16_t* dy;      // bf16 [M, N]
  const int32_t* src_row;  // original row of a slot or null (identity)
  unsigned char* dyp;
  uint32_t M, N, NB, n_row_blocks, n_col_groups;
};

__global__ __launch_bounds__(256) void bwd_pack_dy_kernel(BwdPackDyArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint64_t gid = (uint64_t)blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t q = (uint32_t)(gid & 1u);
  const uint64_t rest = gid >> 1;
  const uint32_t G = (uint32_t)(rest % a.n_col_groups);
  const uint32_t mb = (uint32_t)(rest / a.n_col_groups);
  if (mb >= a.n_row_blocks) return;
  const uint32_t i = lane & 31u, h = lane >> 5;
  const uint32_t p = mb * 32u + i;
  int src = -1;
  if (a.src_row) src = a.src_row[p]; else if (p < a.M) src = (int)p;
  if (src >= (int)a.M) src = -1;
  const uint32_t c0 = 128u * G + 64u * q + 16u * h;
  uint16_t v[2][16];
#pragma unroll
  for (int ch = 0; ch < 2; ++ch) {
    const uint32_t col = c0 + 32u * ch;
    if (src >= 0 && col + 16u <= a.N && (a.N & 7u) == 0) {
      const v8us lo = *reinterpret_cast<const v8us*>(a.dy + (size_t)src * a.N + col);
      const v8us hi = *reinterpret_cast<const v8us*>(a.dy + (size_t)src * a.N + col + 8u);
#pragma unroll
      for (int e = 0; e < 8; ++e) { v[ch][e] = lo[e]; v[ch][8 + e] = hi[e]; }
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) v[ch][e] = (src >= 0 && col + e < a.N) ? a.dy[(size_t)src * a.N + col + e] : (uint16_t)0;
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v8us o;
#pragma unroll
    for (int e = 0; e < 4; ++e) { o[e] = v[0][4 * e + j]; o[4 + e] = v[1][4 * e + j]; }
    const size_t off = ((((size_t)mb * a.NB + 4u * G + j) * 2u + q) * 64u + lane) * 16u;
    *reinterpret_cast<v8us*>(a.dyp + off) = o;
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
};

template <int NKK>
__global__ __launch_bounds__(512, 1) void bwd_dx_kernel(BwdDxArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wrow = wave >> 2, wcol = wave & 3;
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
  const uint32_t per_xcd = (ntile + 7u) / 8u, wgs_per_xcd = gridDim.x >> 3;
  for (uint32_t ti = blockIdx.x >> 3; ti < per_xcd; ti += wgs_per_xcd) {
    const uint32_t t = (blockIdx.x & 7u) * per_xcd + ti;
    if (t >= ntile) break;
    // band-major tile order: 4 row tiles x all k tiles, so an XCD's workgroups share panels
    const uint32_t band = t / (4u * g.tiles_k);
    const uint32_t band_rows = (g.tiles_m - band * 4u) < 4u ? (g.tiles_m - band * 4u) : 4u;
    const uint32_t in_band = t - band * 4u * g.tiles_k;
    const uint32_t tm = band * 4u + in_band % band_rows, tk = in_band / band_rows;

    // this wave's two panel chunks of a stage (row block = wave, halves q = 0, 1) and its weight block
    const unsigned char* Ag = g.dyp + ((size_t)(tm * 8u + (uint32_t)wave) * g.NB) * 2048u + lane * 16;
    const uint32_t kbw = tk * 8u + (uint32_t)wcol * 2u;  // first of the two k blocks this wave multiplies
    const uint32_t kbl = tk * 8u + (uint32_t)wave < g.KB ? tk * 8u + (uint32_t)wave : g.KB - 1u;  // the block it loads
    const unsigned char* Bg = g.wp + (size_t)kbl * kBlockBytes + lane * 16;
    const size_t nb_stride = (size_t)g.KB * kBlockBytes;

    auto issue = [&](int nb) {
      unsigned char* St = lds + (nb % kBwdStages) * kBwdStageBytes;
      const unsigned char* src = Ag + (size_t)nb * 2048u;
      load_1k_to_lds(src, St + (wave * 2) * kBlockBytes);
      load_1k_to_lds(src + 1024, St + (wave * 2 + 1) * kBlockBytes);
      load_1k_to_lds(Bg + (size_t)nb * nb_stride, St + kBwdStagePanel + wave * kBlockBytes);
      // every wave fetches the same 1 KiB of scales (the stage's 32 lead it) to the same place
      load_1k_to_lds(reinterpret_cast<const unsigned char*>(g.swp + 32 * nb) + lane * 16,
                     St + kBwdStagePanel + kBwdStageWeight);
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
      const uint32_t st = lds_base + (nb1 % kBwdStages) * kBwdStageBytes + kBwdStagePanel;
      const uint32_t wa = st + (wcol * 2) * kBlockBytes + lane * 16;
      const uint32_t sa = st + kBwdStageWeight + 16 * h;
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
        acc[rb][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bqC[0][q], acc[rb][0], 0, 0, 0);
        acc[rb][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bqC[1][q], acc[rb][1], 0, 0, 0);
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
    {  // operands of stage 0
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
      const uint32_t pbase = tm * 256u + (uint32_t)wrow * 128u + rb * 32u;
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
// Every group is cut into chunks of 256 rows; chunk c of the call computes, for its rows,
//   partA[c][j][k] = sum_m rs[m][j] * x[m][k]        partB[c][j][n] = sum_m z[m][j] * dy[m][n]
// in float32 (a thread owns two adjacent columns and the whole rank), and a second kernel adds a
// group's chunks in chunk order, scales dB, casts and writes dA [g][K][r], dB [g][r][N], plus
// ds[g] = sum_m sum_j r[m][j] * z[m][j] with r the unscaled dy @ B.T.  Fixed orders: results are
// deterministic.
// ---------------------------------------------------------------------------------------
constexpr uint32_t kBwdChunkRows = 256;
constexpr uint32_t kBwdRankStride = 64;  // floats per slot in the z / r tables

struct BwdDloraArgs {
  const uint16_t* x;        // bf16 [M, K]
  const uint16_t* dy;       // bf16 [M, N]
  const float* rs;          // f32 [slots][64]  (dy @ B.T) * s
  const float* z;           // f32 [slots][64]  x @ A
  const int32_t* src_row;   // or null
  const int32_t* group_off; // [n_groups + 1]
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

template <int R>  // rank padded to 16, 32 or 64
__global__ __launch_bounds__(256) void bwd_dlora_kernel(BwdDloraArgs a) {
  constexpr uint32_t kStageRows = 128;  // rows of the skinny operand staged in LDS at a time
  __shared__ float P[kStageRows][R];
  __shared__ int rowsrc[kStageRows];
  __shared__ uint32_t info[3];
  const uint32_t tid = threadIdx.x;
  const uint32_t per_chunk = a.col_tiles_a + a.col_tiles_b;
  const uint32_t cid = blockIdx.x / per_chunk, ct = blockIdx.x % per_chunk;
  if (tid == 0) {
    uint32_t grp = 0, slot0 = 0, rows = 0;
    if (!bwd_find_chunk(a.group_off, a.n_groups, cid, grp, slot0, rows)) rows = 0;
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
  const uint32_t col = ((job_a ? ct : ct - a.col_tiles_a) * 256u + tid) * 2u;
  const bool active = col < C;  // C is even
  const uint16_t* qcol = Q + (active ? col : 0u);
  float acc0[R], acc1[R];
#pragma unroll
  for (int j = 0; j < R; ++j) { acc0[j] = 0.0f; acc1[j] = 0.0f; }
  for (uint32_t base = 0; base < rows; base += kStageRows) {
    const uint32_t cnt = rows - base < kStageRows ? rows - base : kStageRows;
    __syncthreads();
    for (uint32_t i = tid; i < cnt * R; i += 256u)
      P[i / R][i % R] = psrc[(size_t)(slot0 + base + i / R) * kBwdRankStride + i % R];
    for (uint32_t i = tid; i < cnt; i += 256u)
      rowsrc[i] = a.src_row ? a.src_row[slot0 + base + i] : (int)(slot0 + base + i);
    __syncthreads();
    if (!active) continue;
    uint32_t m = 0;
    for (; m + 4u <= cnt; m += 4u) {
      uint32_t w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) w[u] = *reinterpret_cast<const uint32_t*>(qcol + (size_t)rowsrc[m + u] * C);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float q0 = __uint_as_float(w[u] << 16), q1 = __uint_as_float(w[u] & 0xffff0000u);
#pragma unroll
        for (int j = 0; j < R; ++j) {
          const float pv = P[m + u][j];
          acc0[j] = __builtin_fmaf(pv, q0, acc0[j]);
          acc1[j] = __builtin_fmaf(pv, q1, acc1[j]);
        }
      }
    }
    for (; m < cnt; ++m) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(qcol + (size_t)rowsrc[m] * C);
      const float q0 = __uint_as_float(w << 16), q1 = __uint_as_float(w & 0xffff0000u);
#pragma unroll
      for (int j = 0; j < R; ++j) {
        const float pv = P[m][j];
        acc0[j] = __builtin_fmaf(pv, q0, acc0[j]);
        acc1[j] = __builtin_fmaf(pv, q1, acc1[j]);
      }
    }
  }
  if (!active) return;
#pragma unroll
  for (int j = 0; j < R; ++j)
    *reinterpret_cast<float2*>(part + ((size_t)cid * R + j) * C + col) = make_float2(acc0[j], acc1[j]);
}

struct BwdReduceArgs {
  const float* partA; const float* partB;
  const float* r_raw;       // f32 [slots][64] unscaled dy @ B.T
  const float* z;           // f32 [slots][64]
  const float* lora_scaling;
  const int32_t* group_off;
  uint16_t* d_a;            // bf16 [n_groups, K, r] or null
  uint16_t* d_b;            // bf16 [n_groups, r, N] or null
  float* d_s;               // f32 [n_groups] or null
  uint32_t K, N, r, R, n_groups, blocks_a, blocks_b;
};

__global__ __launch_bounds__(256) void bwd_dlora_reduce_kernel(BwdReduceArgs a) {
  __shared__ uint32_t chunk0[kMaxAdapters + 1];
  __shared__ double red[256];
  const uint32_t tid = threadIdx.x;
  if (tid == 0) {
    uint32_t run = 0;
    for (uint32_t gq = 0; gq < a.n_groups; ++gq) {
      chunk0[gq] = run;
      run += ((uint32_t)(a.group_off[gq + 1] - a.group_off[gq]) + kBwdChunkRows - 1u) / kBwdChunkRows;
    }
    chunk0[a.n_groups] = run;
  }
  __syncthreads();
  uint32_t b = blockIdx.x;
  if (b < a.blocks_a + a.blocks_b) {
    const bool job_a = b < a.blocks_a;
    const uint32_t C = job_a ? a.K : a.N;
    const uint64_t e = (uint64_t)(job_a ? b : b - a.blocks_a) * 256u + tid;  // (group, j, column), column fastest
    if (e >= (uint64_t)a.n_groups * a.r * C) return;
    const uint32_t col = (uint32_t)(e % C);
    const uint32_t j = (uint32_t)((e / C) % a.r), grp = (uint32_t)(e / ((uint64_t)C * a.r));
    const float* part = job_a ? a.partA : a.partB;
    float sum = 0.0f;
    for (uint32_t ch = chunk0[grp]; ch < chunk0[grp + 1]; ++ch) sum += part[((size_t)ch * a.R + j) * C + col];
    if (job_a) {
      if (a.d_a) a.d_a[((size_t)grp * a.K + col) * a.r + j] = (uint16_t)f32_to_bf16_bits(sum);
    } else {
      if (a.d_b) a.d_b[((size_t)grp * a.r + j) * a.N + col] = (uint16_t)f32_to_bf16_bits(sum * a.lora_scaling[grp]);
    }
    return;
  }
  b -= a.blocks_a + a.blocks_b;  // one block per group: ds
  if (b >= a.n_groups || !a.d_s) return;
  const uint32_t o0 = (uint32_t)a.group_off[b], o1 = (uint32_t)a.group_off[b + 1];
  double sum = 0.0;
  for (uint32_t i = o0 * a.r + tid; i < o1 * a.r; i += 256u) {
    const uint32_t slot = i / a.r, j = i % a.r;
    sum += (double)a.r_raw[(size_t)slot * kBwdRankStride + j] * (double)a.z[(size_t)slot * kBwdRankStride + j];
  }
  red[tid] = sum;
  __syncthreads();
  for (uint32_t o = 128; o > 0; o >>= 1) {
    if (tid < o) red[tid] += red[tid + o];
    __syncthreads();
  }
  if (tid == 0) a.d_s[b] = (float)red[0];
}

}  // namespace w8a8
