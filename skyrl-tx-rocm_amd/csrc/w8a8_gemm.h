// Tiled int8 MFMA GEMM with the fused float32 epilogue:
//   acc[p, n]  = sum_k xq[p, k] * wq[k, n]                         (v_mfma_i32_32x32x32_i8, exact)
//   base       = (float(acc) * sx[p]) * sw[n]                      (skyrl/tx/kernels/quantized_lora.py:248-252)
//   y          = base + low * s[group(p)] (+ residual)             (quantized_lora.py:300-304)
//   low        = z[p, :] @ B[group(p)]                             (bf16 MFMA, z carried as 3 (or 2) bf16 terms)
//   out        = bf16(y)   or   bf16(silu(bf16(y_gate)) * bf16(y_up))
// Workgroup = 256 threads = 4 waves stacked along M (64 x 128 each), tile 256 x 128, 128
// accumulator registers per lane and 72 KiB of LDS, so two workgroups share a CU: while one is
// in its VALU/store epilogue the other keeps the MFMA pipe busy.  K is consumed in steps of 64
// through a ring of three 24 KiB LDS stages filled by 16-byte direct-to-LDS loads of contiguous
// 1 KiB fragment blocks, two tiles ahead of the MFMAs.
#pragma once
#include <type_traits>

#include "w8a8_device.h"

namespace w8a8 {

enum { kEpiPlain = 0, kEpiSwiglu = 1, kEpiAcc = 2 };

struct GemmArgs {
  const unsigned char* xq;   // packed activation codes [slots, K_pad]
  const unsigned char* wp;   // packed weight [N_pad, K_pad]
  const float* sx;           // f32 [slots]
  const float* sw;           // f32 [N]
  const unsigned char* zp;   // packed z fragments [slots/32][NKK][3][64 lanes][8 bf16] or null
  const uint16_t* lora_b;    // bf16 [n_groups, rank, N] or null
  const float* lora_scaling; // f32 [n_groups]
  const int32_t* src_row;    // original row of every grouped slot, or null (identity)
  const int32_t* slot_group; // LoRA group (adapter) of every grouped slot, or null (group 0)
  const int32_t* blk_range;  // per 32-row block: first group | last group << 16, or null
  const uint16_t* residual;  // bf16 [M, n_out] or null
  void* out;                 // bf16 [M, n_out] or int32 [M, N]
  uint64_t w_group_stride;   // grouped mode: bytes between the packed weights of two experts
  uint32_t M, N, K_pad, KB, slots, total_rows;
  uint32_t tiles_m, tiles_n, rank, nsplit_terms, map_mode;
  uint32_t groups_per_weight; // grouped mode: weight index = group / groups_per_weight
};

// float32 pair -> packed bf16x2 (round to nearest even, v_cvt_pk_bf16_f32)
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf));
}

// silu(g) * u with g, u already rounded to bf16 (x * logistic(x), exp and reciprocal in
// hardware precision: 1 ulp each)
__device__ inline float swiglu_f32(float g, float u) {
  const float sig = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
  return (g * sig) * u;
}

constexpr int kGemmTileM = 256;
constexpr int kGemmTileN = 128;
constexpr int kGemmStages = 3;
constexpr int kGemmStageBytes = 24576;  // A: 8 row blocks x 2 k blocks, B: 4 column blocks x 2 k blocks
constexpr int kGemmLdsBytes = kGemmStages * kGemmStageBytes;
// Grouped (ragged, per-expert weight) mode: tile 64 x 512, the four waves sit side by side along
// N (64 x 128 each) and share the 64-row activation panel; every 64-row tile belongs to one group.
constexpr int kGroupedTileM = 64;
constexpr int kGroupedTileN = 512;
constexpr int kGroupedStages = 4;
constexpr int kGroupedStageBytes = 36864;  // A: 2 row blocks x 2 k blocks, B: 16 column blocks x 2 k blocks
constexpr int kGroupedLdsBytes = kGroupedStages * kGroupedStageBytes;

template <int EPI, int NKK, int DBG = 0, bool GROUPED = false>
__global__ __launch_bounds__(256, GROUPED ? 1 : 2) void w8a8_gemm_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- XCD-aware tile mapping: consecutive workgroup ids land on different XCDs, so each
  // XCD gets a contiguous range of a band-major tile order (GM row tiles x all column tiles).
  const uint32_t total_rows = g.total_rows;
  const uint32_t ntile = g.tiles_m * g.tiles_n;
  const uint32_t per_xcd = (ntile + 7u) / 8u;
  const uint32_t t = g.map_mode == 1 ? blockIdx.x : (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
  if (t >= ntile) return;
  constexpr uint32_t GM = GROUPED ? 1 : 4;
  const uint32_t band = t / (GM * g.tiles_n);
  const uint32_t band_rows = (g.tiles_m - band * GM) < GM ? (g.tiles_m - band * GM) : GM;
  const uint32_t in_band = t - band * GM * g.tiles_n;
  const uint32_t tm = band * GM + in_band % band_rows;
  const uint32_t tn = in_band / band_rows;

  constexpr uint32_t kRowBlocks = GROUPED ? 2 : 8;   // 32-row blocks of the activation panel
  constexpr uint32_t kColBlocks = GROUPED ? 16 : 4;  // 32-column blocks of the weight panel
  uint32_t tile_group = 0;
  if (GROUPED) {
    const int32_t range = g.blk_range[tm * 2u];
    if (range < 0) return;  // tile beyond the rows in use
    tile_group = (uint32_t)range & 0xffffu;
  }
  const uint32_t widx = GROUPED ? tile_group / g.groups_per_weight : 0u;
  const uint32_t ncb_total = n_padded(g.N) / 32u;  // column blocks of the packed weight
  const unsigned char* Ag = g.xq + (size_t)tm * kRowBlocks * g.KB * kBlockBytes;
  const unsigned char* Bg = g.wp + (size_t)widx * g.w_group_stride;
  const float* swp = g.sw + (size_t)widx * (GROUPED ? g.N : 0u);

  v16i acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // ---- main loop
  constexpr int kStages = GROUPED ? kGroupedStages : kGemmStages;
  constexpr int kStageBytes = GROUPED ? kGroupedStageBytes : kGemmStageBytes;
  constexpr int kAChunks = kRowBlocks * 2;                    // 1 KiB chunks of A per stage
  constexpr int kLoadsPerTile = (kAChunks + kColBlocks * 2) / 4;  // direct-to-LDS loads per wave per tile
  const int KT = (int)(g.K_pad / 64u);
  auto issue = [&](int kt) {
    unsigned char* St = lds + (kt % kStages) * kStageBytes;
#pragma unroll
    for (int q = 0; q < kLoadsPerTile; ++q) {
      const int c = wave * kLoadsPerTile + q;  // chunks < kAChunks: A (row block c/2, k block c%2); then B
      const bool isA = c < kAChunks;
      uint32_t rb = isA ? (uint32_t)(c >> 1) : tn * kColBlocks + (uint32_t)((c - kAChunks) >> 1);
      if (!isA && rb >= ncb_total) rb = ncb_total - 1u;  // keep every wave's load count equal
      const unsigned char* base = isA ? Ag : Bg;
      const size_t goff = ((size_t)rb * g.KB + (size_t)kt * 2 + (c & 1)) * kBlockBytes + lane * 16;
      load_1k_to_lds(base + goff, St + c * kBlockBytes);
    }
  };
  auto read_frags = [&](int kt, int ks, v4i (&af)[2], v4i (&bf)[4]) {
    const unsigned char* As = lds + (kt % kStages) * kStageBytes;
    const unsigned char* Bs = As + kAChunks * kBlockBytes;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      af[i] = *reinterpret_cast<const v4i*>(As + (((GROUPED ? 0 : wave * 2) + i) * 2 + ks) * kBlockBytes + lane * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      bf[j] = *reinterpret_cast<const v4i*>(Bs + (((GROUPED ? wave * 4 : 0) + j) * 2 + ks) * kBlockBytes + lane * 16);
  };
  auto mfma8 = [&](const v4i (&af)[2], const v4i (&bf)[4]) {
    if constexpr (DBG == 1) {  // measurement only: no MFMA work, keep the operands alive
#pragma unroll
      for (int i = 0; i < 2; ++i) asm volatile("" ::"v"(af[i]), "v"(bf[i]), "v"(bf[i + 2]));
      return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
  };

  v4i fa0[2], fb0[4], fa1[2], fb1[4];
#pragma unroll
  for (int st = 0; st < kStages - 1; ++st)
    if (st < KT) issue(st);
  if (KT > kStages - 2) wait_vmcnt<(kStages - 2) * kLoadsPerTile>(); else wait_vmcnt<0>();
  lds_barrier();
  read_frags(0, 0, fa0, fb0);
  const int KT_main = KT - (kStages - 1);  // tiles that still have a tile to prefetch
  int kt = 0;
  for (; kt < KT_main; ++kt) {
    // ---- k-step 0 of tile kt: prefetch the k-step 1 fragments and the tile kStages-1 ahead.
    // The MFMAs lead so that the wait for their operands does not cover the new LDS reads.
    read_frags(kt, 1, fa1, fb1);
    if constexpr (DBG < 2) issue(kt + kStages - 1);
    mfma8(fa0, fb0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // 1 VMEM read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- k-step 1: tile kt+1 must have landed before its first fragments are fetched
    if constexpr (DBG < 2) wait_vmcnt<(kStages - 2) * kLoadsPerTile>();
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(kt + 1, 0, fa0, fb0);
    mfma8(fa1, fb1);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (; kt < KT; ++kt) {  // drain: nothing left to prefetch
    read_frags(kt, 1, fa1, fb1);
    mfma8(fa0, fb0);
    wait_vmcnt<0>();
    lds_barrier();
    if (kt + 1 < KT) read_frags(kt + 1, 0, fa0, fb0);
    mfma8(fa1, fb1);
  }
  lds_barrier();  // every wave is done with the stage buffers; the epilogue reuses the LDS

  // ------------------------------------------------------------------ epilogue
  // Lane (c = lane % 32, h = lane / 32) owns, in each of its wave's two 32 x 128 strips, the four
  // consecutive original columns ncol .. ncol+3 (accumulator blocks j = 0..3) of the 16 rows
  // 8*(v/4) + 4*h + v%4.
  constexpr bool kLora = (NKK > 0) && (EPI != kEpiAcc);
  constexpr int kZ = NKK > 0 ? NKK : 1;
  const int c = lane & 31, h = lane >> 5;
  const uint32_t m0 = GROUPED ? tm * 64u : tm * 256u + wave * 64u;
  const uint32_t tcol0 = GROUPED ? tn * 512u + wave * 128u : tn * 128u;  // first column of the wave
  const uint32_t ncol = tcol0 + 4u * c;
  const uint32_t n_out = (EPI == kEpiSwiglu) ? g.N / 2u : g.N;
  const bool full_n = (tcol0 + 128u <= g.N) && ((g.N & 3u) == 0);  // wave-uniform
  if (GROUPED && tcol0 >= g.N) return;  // wave beyond the last column (after the last barrier)
  float sw[4] = {0.f, 0.f, 0.f, 0.f};
  if (EPI != kEpiAcc) {
    if (full_n) {
      const float4 s4 = *reinterpret_cast<const float4*>(swp + ncol);
      sw[0] = s4.x; sw[1] = s4.y; sw[2] = s4.z; sw[3] = s4.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (ncol + j < g.N) sw[j] = swp[ncol + j];
    }
  }
  // LoRA-B staging, private to the wave: bf16 [16*NKK][128] at lds + wave * 16 KiB
  uint16_t* Bl = reinterpret_cast<uint16_t*>(lds + wave * 16384);
  int staged = -1;

  auto load_zfrags = [&](uint32_t blk, v8us (&zf)[kZ][3]) {
    if constexpr (kLora) {
      const unsigned char* zb = g.zp + (size_t)blk * NKK * 3u * kBlockBytes + lane * 16;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
        for (int s = 0; s < 3; ++s)
          zf[kk][s] = *reinterpret_cast<const v8us*>(zb + (kk * 3 + s) * kBlockBytes);
    }
  };

  auto epilogue_block = [&](auto BI) {
    constexpr int bi = decltype(BI)::value;
    const uint32_t pbase = m0 + bi * 32u;
    if (pbase >= total_rows) return;  // wave-uniform
    const uint32_t blk = pbase / 32u;
    if (GROUPED && g.blk_range[blk] < 0) return;  // block beyond the rows in use
    v8us zf[kZ][3];
    load_zfrags(blk, zf);

    // rows this lane owns in the block: 8*gq + 4*h + e
    float sxv[16];
    uint32_t rowoff[16];  // element offset of the output row, or 0xffffffff for padding rows
    bool all_rows = true;
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const uint32_t p4 = pbase + 8u * gq + 4u * h;
      if (EPI != kEpiAcc) {
        const float4 s4 = *reinterpret_cast<const float4*>(g.sx + p4);
        sxv[4 * gq + 0] = s4.x; sxv[4 * gq + 1] = s4.y; sxv[4 * gq + 2] = s4.z; sxv[4 * gq + 3] = s4.w;
      }
      int src[4];
      if (g.src_row) {
        const int4 r4 = *reinterpret_cast<const int4*>(g.src_row + p4);
        src[0] = r4.x; src[1] = r4.y; src[2] = r4.z; src[3] = r4.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) src[e] = (int)(p4 + e);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool ok = src[e] >= 0 && src[e] < (int)g.M;
        all_rows = all_rows && ok;
        rowoff[4 * gq + e] = ok ? (uint32_t)src[e] * ((EPI == kEpiAcc) ? g.N : n_out) : 0xffffffffu;
      }
    }
    const bool fast = full_n && (__builtin_amdgcn_ballot_w64(!all_rows) == 0);  // uniform

    if (EPI == kEpiAcc) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if (!fast && rowoff[v] == 0xffffffffu) continue;
        int32_t* o = reinterpret_cast<int32_t*>(g.out) + rowoff[v] + ncol;
        if (fast) {
          *reinterpret_cast<int4*>(o) = make_int4(acc[bi][0][v], acc[bi][1][v], acc[bi][2][v], acc[bi][3][v]);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (ncol + j < g.N) o[j] = acc[bi][j][v];
        }
      }
      return;
    }

    float y[16][4];
#pragma unroll
    for (int v = 0; v < 16; ++v)
#pragma unroll
      for (int j = 0; j < 4; ++j) y[v][j] = ((float)acc[bi][j][v] * sxv[v]) * sw[j];

    if constexpr (kLora) {
      // groups (adapters) present in this 32-row block: usually one, two at a group boundary
      const uint32_t range = g.blk_range ? (uint32_t)g.blk_range[blk] : 0u;
      const int glo = (int)(range & 0xffffu), ghi = (int)(range >> 16);
      const int rowgrp = (g.slot_group && ghi > glo) ? g.slot_group[pbase + c] : glo;
      for (int gi = glo; gi <= ghi; ++gi) {  // wave-uniform
        if (gi != staged) {
          // stage B[gi][0:16*NKK][tile columns] as bf16 [16*NKK][128]; LDS operations of one
          // wave execute in order, so no barrier is needed around this wave-private buffer
          const uint16_t* Bsrc = g.lora_b + (size_t)gi * g.rank * g.N;
          for (uint32_t q = (uint32_t)lane; q < NKK * 16u * 16u; q += 64u) {
            const uint32_t r = q >> 4, cc = (q & 15u) * 8u;
            v8us val = {0, 0, 0, 0, 0, 0, 0, 0};
            if (r < g.rank) {
              const size_t off = (size_t)r * g.N + tcol0 + cc;
              if ((g.N & 7u) == 0 && tcol0 + cc + 8u <= g.N) {
                val = *reinterpret_cast<const v8us*>(Bsrc + off);
              } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  if (tcol0 + cc + e < g.N) val[e] = Bsrc[off + e];
              }
            }
            *reinterpret_cast<v8us*>(Bl + r * 128u + cc) = val;
          }
          staged = gi;
        }
        const bool mine = (ghi == glo) || (rowgrp == gi);
        const float sgrp = g.lora_scaling[gi];
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
          v16f low[2];
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) low[j][e] = 0.0f;
#pragma unroll
          for (int kk = 0; kk < NKK; ++kk) {
            const v8us zero = {0, 0, 0, 0, 0, 0, 0, 0};
            const v8us z0 = mine ? zf[kk][0] : zero, z1 = mine ? zf[kk][1] : zero, z2 = mine ? zf[kk][2] : zero;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              v8us bfr;
              const uint32_t col = 4u * c + 2u * jp + j;
#pragma unroll
              for (int e = 0; e < 8; ++e) bfr[e] = Bl[(16u * kk + 8u * h + e) * 128u + col];
              const v8bf bb = __builtin_bit_cast(v8bf, bfr);
              if (g.nsplit_terms >= 3)
                low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, z2), bb, low[j], 0, 0, 0);
              low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, z1), bb, low[j], 0, 0, 0);
              low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, z0), bb, low[j], 0, 0, 0);
            }
          }
#pragma unroll
          for (int v = 0; v < 16; ++v)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const float l = low[j][v] * sgrp;
              y[v][2 * jp + j] = y[v][2 * jp + j] + l;
            }
        }
      }
    }

#pragma unroll
    for (int v = 0; v < 16; ++v) {
      if (!fast && rowoff[v] == 0xffffffffu) continue;
      if (EPI == kEpiSwiglu) {
        // (y0, y1) and (y2, y3) are (gate, up) of the product columns ncol/2 and ncol/2 + 1
        const uint32_t f01 = pack_bf16x2(y[v][0], y[v][1]), f23 = pack_bf16x2(y[v][2], y[v][3]);
        const float p0 = swiglu_f32(__uint_as_float(f01 << 16), __uint_as_float(f01 & 0xffff0000u));
        const float p1 = swiglu_f32(__uint_as_float(f23 << 16), __uint_as_float(f23 & 0xffff0000u));
        uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + rowoff[v] + (ncol >> 1);
        const uint32_t pk = pack_bf16x2(p0, p1);
        if (fast) {
          *reinterpret_cast<uint32_t*>(o) = pk;
        } else {
          if ((ncol >> 1) < n_out) o[0] = (uint16_t)(pk & 0xffffu);
          if ((ncol >> 1) + 1u < n_out) o[1] = (uint16_t)(pk >> 16);
        }
      } else {
        uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + rowoff[v] + ncol;
        if (fast) {
          float r0 = y[v][0], r1 = y[v][1], r2 = y[v][2], r3 = y[v][3];
          if (g.residual) {
            const uint2 rr = *reinterpret_cast<const uint2*>(g.residual + rowoff[v] + ncol);
            r0 = r0 + __uint_as_float(rr.x << 16);
            r1 = r1 + __uint_as_float(rr.x & 0xffff0000u);
            r2 = r2 + __uint_as_float(rr.y << 16);
            r3 = r3 + __uint_as_float(rr.y & 0xffff0000u);
          }
          *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf16x2(r0, r1), pack_bf16x2(r2, r3));
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (ncol + j < g.N) {
              float yy = y[v][j];
              if (g.residual) yy = yy + bf16_bits_to_f32(g.residual[rowoff[v] + ncol + j]);
              o[j] = (uint16_t)(pack_bf16x2(yy, 0.0f) & 0xffffu);
            }
          }
        }
      }
    }
  };
  epilogue_block(std::integral_constant<int, 0>{});
  epilogue_block(std::integral_constant<int, 1>{});
}

}  // namespace w8a8
