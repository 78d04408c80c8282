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
  const float* lora_scaling; // f32 [n_groups]
  const unsigned char* bp;   // LoRA B in MFMA operand order [n_groups][N_pad/32][NKK][64 lanes][8 bf16] or null
  const int32_t* src_row;    // original row of every grouped slot, or null (identity)
  const int32_t* slot_group; // LoRA group (adapter) of every grouped slot, or null (group 0)
  const int32_t* blk_range;  // per 32-row block: first group | last group << 16, or null
  const uint16_t* residual;  // bf16 [M, n_out] or null
  void* out;                 // bf16 [M, n_out] or int32 [M, N]
  uint64_t w_group_stride;   // grouped mode: bytes between the packed weights of two experts
  uint32_t M, N, K_pad, KB, slots, total_rows;
  uint32_t tiles_m, tiles_n, rank;
  uint32_t groups_per_weight; // grouped mode: weight index = group / groups_per_weight
  uint32_t* tile_ctr;         // 8 zeroed counters, 64 bytes apart (one per XCD), or null: static schedule
};

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
// grouped geometry for experts with many rows: 128 x 512 tile, 8 waves (2 x 4), the weight panel
// travels L2 -> LDS once per 128 rows instead of once per 64
constexpr int kGrouped128TileM = 128;
constexpr int kGrouped128Stages = 3;
constexpr int kGrouped128StageBytes = 40960;  // A: 4 row blocks x 2 k blocks, B: 16 column blocks x 2 k blocks
constexpr int kGrouped128LdsBytes = kGrouped128Stages * kGrouped128StageBytes;

// (The 256 x 256 geometry for large problems is a kernel of its own: w8a8_gemm16.h.)
// Dense geometry for calls whose 256 x 128 tiles would leave most CUs idle: 128 x 128 tiles, the four
// waves stacked along M with 32 x 128 each, so a wave carries half the MFMAs and half the epilogue.
constexpr int kGemm128TileM = 128;
constexpr int kGemm128StageBytes = 16384;  // A: 4 row blocks x 2 k blocks, B: 4 column blocks x 2 k blocks
enum { kModeDense = 0, kModeGrouped = 1, kModeGrouped128 = 2, kModeDense128 = 3 };

// One tile of the persistent loop.
struct GemmTile {
  const unsigned char* Ag;  // packed activation panel of the tile
  const unsigned char* Bg;  // packed weight of the tile's group
  const float* swp;         // per-channel scales of the tile's group
  uint32_t tm, tn;
  bool valid;
};

template <int EPI, int NKK, int MODE = kModeDense>
__global__ __launch_bounds__(MODE == kModeGrouped128 ? 512 : 256, (MODE == kModeDense || MODE == kModeDense128) ? 2 : 1)
void w8a8_gemm_kernel(GemmArgs g) {
  constexpr bool G128 = MODE == kModeGrouped128;
  constexpr bool D128 = MODE == kModeDense128;
  constexpr bool GROUPED = MODE == kModeGrouped || G128;
  constexpr int kWaves = G128 ? 8 : 4;
  constexpr int kWR = D128 ? 1 : 2;                                  // 32-row blocks of a wave's tile
  constexpr uint32_t kRowBlocks = (G128 || D128) ? 4 : (GROUPED ? 2 : 8);  // 32-row blocks of the activation panel
  constexpr uint32_t kColBlocks = GROUPED ? 16 : 4;                 // 32-column blocks of the weight panel
  constexpr int kStages = G128 ? kGrouped128Stages : (GROUPED ? kGroupedStages : kGemmStages);
  constexpr int kStageBytes =
      G128 ? kGrouped128StageBytes : (GROUPED ? kGroupedStageBytes : (D128 ? kGemm128StageBytes : kGemmStageBytes));
  constexpr int kAChunks = kRowBlocks * 2;                              // 1 KiB chunks of A per stage
  constexpr int kLoadsPerTile = (kAChunks + kColBlocks * 2) / kWaves;   // direct-to-LDS loads per wave per k-tile
  constexpr bool kLora = (NKK > 0) && (EPI != kEpiAcc);

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wrow = G128 ? (wave >> 2) : (GROUPED ? 0 : wave);  // wave position along M (32 * kWR rows each)
  const int wcol = G128 ? (wave & 3) : (GROUPED ? wave : 0);    // wave position along N (128 columns each)
  const int c = lane & 31, h = lane >> 5;

  const uint32_t total_rows = g.total_rows;
  const uint32_t ntile = g.tiles_m * g.tiles_n;
  const uint32_t ncb_total = n_padded(g.N) / 32u;  // column blocks of the packed weight
  const uint32_t n_out = (EPI == kEpiSwiglu) ? g.N / 2u : g.N;
  const int KT = (int)(g.K_pad / 64u);

  // ---- persistent tile schedule.  Consecutive workgroup ids land on different XCDs, so each XCD
  // walks a contiguous range of a band-major tile order (GM row tiles x all column tiles) and the
  // workgroups of an XCD work on neighbouring tiles at any time (shared panels hit in its L2).
  const uint32_t per_xcd = (ntile + 7u) / 8u;
  const uint32_t wgs_per_xcd = gridDim.x >> 3;
  // `i` is a position inside the XCD's range of the tile order.
  auto tile_at = [&](uint32_t i) -> GemmTile {
    GemmTile T{};
    const uint32_t t = i < per_xcd ? (blockIdx.x & 7u) * per_xcd + i : ntile;
    if (t >= ntile) return T;
    constexpr uint32_t GM = GROUPED ? 1 : 4;
    const uint32_t band = t / (GM * g.tiles_n);
    const uint32_t band_rows = (g.tiles_m - band * GM) < GM ? (g.tiles_m - band * GM) : GM;
    const uint32_t in_band = t - band * GM * g.tiles_n;
    T.tm = band * GM + in_band % band_rows;
    T.tn = in_band / band_rows;
    uint32_t widx = 0;
    if (GROUPED) {
      const int32_t range = g.blk_range[T.tm * kRowBlocks];
      if (range < 0) return T;  // tile beyond the rows in use: nothing to do, but later tiles may exist
      widx = ((uint32_t)range & 0xffffu) / g.groups_per_weight;
    }
    T.Ag = g.xq + (size_t)T.tm * kRowBlocks * g.KB * kBlockBytes;
    T.Bg = g.wp + (size_t)widx * g.w_group_stride;
    T.swp = g.sw + (size_t)widx * (GROUPED ? g.N : 0u);
    T.valid = true;
    return T;
  };
  // Static schedule: position (workgroup index inside the XCD) + step * (workgroups per XCD).
  // Dynamic schedule (two workgroups per CU): positions come from the XCD's counter, because the
  // hardware favours the older workgroup of a CU and a static split would leave the younger one
  // to finish alone.  The result does not depend on which workgroup computes which tile.
  const bool dyn = !GROUPED && g.tile_ctr != nullptr;
  uint32_t* const ctr = g.tile_ctr + (blockIdx.x & 7u) * 16u;
  __shared__ uint32_t dyn_slot[2];
  uint32_t cur_i = blockIdx.x >> 3, nxt_i = 0;
  if (dyn) {
    if (tid == 0) dyn_slot[0] = atomicAdd(ctr, 1u);
    __syncthreads();
    cur_i = dyn_slot[0];
  }

  auto issue = [&](const GemmTile& T, int kt) {
    unsigned char* St = lds + (kt % kStages) * kStageBytes;
#pragma unroll
    for (int q = 0; q < kLoadsPerTile; ++q) {
      const int ch = wave * kLoadsPerTile + q;  // chunks < kAChunks: A (row block ch/2, k block ch%2); then B
      const bool isA = ch < kAChunks;
      uint32_t rb = isA ? (uint32_t)(ch >> 1) : T.tn * kColBlocks + (uint32_t)((ch - kAChunks) >> 1);
      if (!isA && rb >= ncb_total) rb = ncb_total - 1u;  // keep every wave's load count equal
      const unsigned char* base = isA ? T.Ag : T.Bg;
      const size_t goff = ((size_t)rb * g.KB + (size_t)kt * 2 + (ch & 1)) * kBlockBytes + lane * 16;
      load_1k_to_lds(base + goff, St + ch * kBlockBytes);
    }
  };
  auto read_frags = [&](int kt, int ks, v4i (&af)[kWR], v4i (&bf)[4]) {
    const unsigned char* As = lds + (kt % kStages) * kStageBytes;
    const unsigned char* Bs = As + kAChunks * kBlockBytes;
#pragma unroll
    for (int i = 0; i < kWR; ++i)
      af[i] = *reinterpret_cast<const v4i*>(As + ((wrow * kWR + i) * 2 + ks) * kBlockBytes + lane * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      bf[j] = *reinterpret_cast<const v4i*>(Bs + ((wcol * 4 + j) * 2 + ks) * kBlockBytes + lane * 16);
  };

  bool prefetched = false;  // the first kStages-1 k-tiles of the current tile are already in flight
  for (uint32_t step = 0; cur_i < per_xcd; ++step, cur_i = nxt_i) {
    const GemmTile T = tile_at(cur_i);
    nxt_i = cur_i + wgs_per_xcd;
    if (!T.valid) { prefetched = false; continue; }  // static schedules only (empty grouped tile, range end)

    v16i acc[kWR][4];
#pragma unroll
    for (int i = 0; i < kWR; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    auto mfma8 = [&](const v4i (&af)[kWR], const v4i (&bf)[4]) {
#pragma unroll
      for (int i = 0; i < kWR; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    };

    // ---- main loop
    v4i fa0[kWR], fb0[4], fa1[kWR], fb1[4];
    if (!prefetched) {
#pragma unroll
      for (int st = 0; st < kStages - 1; ++st)
        if (st < KT) issue(T, st);
      if (KT > kStages - 2) wait_vmcnt<(kStages - 2) * kLoadsPerTile>(); else wait_vmcnt<0>();
    } else {
      wait_vmcnt<0>();  // prefetch of this tile and the previous tile's stores
    }
    lds_barrier();
    uint32_t grabbed = 0;  // next position of a dynamic schedule; it arrives during the main loop
    if (dyn && tid == 0) grabbed = atomicAdd(ctr, 1u);
    read_frags(0, 0, fa0, fb0);
    const int KT_main = KT - (kStages - 1);  // k-tiles that still have a k-tile to prefetch
    int kt = 0;
    for (; kt < KT_main; ++kt) {
      // ---- k-step 0 of k-tile kt: prefetch the k-step 1 fragments and the k-tile kStages-1 ahead.
      // The MFMAs lead so that the wait for their operands does not cover the new LDS reads.
      read_frags(kt, 1, fa1, fb1);
      issue(T, kt + kStages - 1);
      mfma8(fa0, fb0);
      if constexpr (kWR == 2) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
#pragma unroll
        for (int q = 0; q < 6; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // 1 VMEM read
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- k-step 1: k-tile kt+1 must have landed before its first fragments are fetched
      wait_vmcnt<(kStages - 2) * kLoadsPerTile>();
      lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
      read_frags(kt + 1, 0, fa0, fb0);
      mfma8(fa1, fb1);
      if constexpr (kWR == 2) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
        for (int q = 0; q < 6; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
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
    if (dyn && tid == 0) dyn_slot[(step + 1u) & 1u] = grabbed;  // the drain loop has waited for it
    lds_barrier();  // every wave is done with the stage buffers
    if (dyn) nxt_i = dyn_slot[(step + 1u) & 1u];

    // ---- the next tile's first k-tiles travel while this tile's epilogue runs (no LDS below)
    prefetched = false;
    if (nxt_i < per_xcd) {
      const GemmTile Tn = tile_at(nxt_i);
      if (Tn.valid) {
#pragma unroll
        for (int st = 0; st < kStages - 1; ++st)
          if (st < KT) issue(Tn, st);
        prefetched = true;
      }
    }

    // ---------------------------------------------------------------- epilogue
    // Lane (c = lane % 32, h = lane / 32) owns, in each of its wave's two 32 x 128 strips, the four
    // consecutive original columns ncol .. ncol+3 (accumulator blocks j = 0..3) of the 16 rows
    // 8*(v/4) + 4*h + v%4.
    const uint32_t m0 = T.tm * (kRowBlocks * 32u) + wrow * (32u * kWR);
    const uint32_t tcol0 = T.tn * (kColBlocks * 32u) + wcol * 128u;  // first column of the wave
    const uint32_t ncol = tcol0 + 4u * c;
    const bool full_n = (tcol0 + 128u <= g.N) && ((g.N & 3u) == 0);  // wave-uniform
    if (tcol0 >= g.N) continue;  // wave beyond the last column; it still takes part in the next tile
    float sw[4] = {0.f, 0.f, 0.f, 0.f};
    if (EPI != kEpiAcc) {
      if (full_n) {
        const float4 s4 = *reinterpret_cast<const float4*>(T.swp + ncol);
        sw[0] = s4.x; sw[1] = s4.y; sw[2] = s4.z; sw[3] = s4.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (ncol + j < g.N) sw[j] = T.swp[ncol + j];
      }
    }
    auto epilogue_block = [&](auto BI) {
      constexpr int bi = decltype(BI)::value;
      const uint32_t pbase = m0 + bi * 32u;
      if (pbase >= total_rows) return;  // wave-uniform
      const uint32_t blk = pbase / 32u;
      if (GROUPED && g.blk_range[blk] < 0) return;  // block beyond the rows in use
      __builtin_amdgcn_sched_barrier(0);  // keep the blocks' register lifetimes apart

      // Per-row scale and output offset of the block's 32 rows live in one register each (lane l
      // holds row l % 32); a lane's 16 rows 8*(v/4) + 4*h + v%4 are fetched across lanes below.
      const float sx_lane = (EPI != kEpiAcc) ? g.sx[pbase + c] : 0.0f;
      const int src_lane = g.src_row ? g.src_row[pbase + c] : (int)(pbase + c);
      const bool row_ok = src_lane >= 0 && src_lane < (int)g.M;
      const uint32_t off_lane = row_ok ? (uint32_t)src_lane * ((EPI == kEpiAcc) ? g.N : n_out) : 0xffffffffu;
      const bool fast = full_n && (__builtin_amdgcn_ballot_w64(!row_ok) == 0);  // wave-uniform
      const int row_addr = 16 * h;  // byte address (4 * lane) of the lane holding row 4*h

      if (EPI == kEpiAcc) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const uint32_t rowoff =
              (uint32_t)__builtin_amdgcn_ds_bpermute(row_addr + 4 * (8 * (v >> 2) + (v & 3)), (int)off_lane);
          if (!fast && rowoff == 0xffffffffu) continue;
          int32_t* o = reinterpret_cast<int32_t*>(g.out) + rowoff + ncol;
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

      // Groups (adapters) present in this 32-row block: one, except at a group boundary.  A
      // boundary block is simply processed once per group; each pass stores only its own rows.
      const uint32_t range = (kLora && g.blk_range) ? (uint32_t)g.blk_range[blk] : 0u;
      const int glo = (int)(range & 0xffffu), ghi = (int)(range >> 16);
      const int grp_lane = (kLora && g.slot_group && ghi > glo) ? g.slot_group[pbase + c] : glo;
      for (int gi = glo; gi <= ghi; ++gi) {  // wave-uniform
      // The lane's four columns are processed as two pairs (jp): LoRA MFMAs of the pair (section A),
      // then dequantize + add + activate per row (section B).  The first pair's packed result waits
      // in `hold` so that every row is written with one 4- or 8-byte store.
      uint32_t hold[16];
#pragma unroll
      for (int jp = 0; jp < 2; ++jp) {
        // ---- section A: lowS[j][v] = s_g * (z @ B_g) for the column pair
        v16f lowS[2];
        if constexpr (kLora) {
          const unsigned char* zb = g.zp + (size_t)blk * NKK * 3u * kBlockBytes + lane * 16;
          // operand of packed column block cb = tcol0/32 + j: rows 16kk + 8h + 0..7 of column 4c + j
          const unsigned char* bb0 =
              g.bp + ((size_t)gi * ncb_total + tcol0 / 32u + 2u * jp) * NKK * kBlockBytes + lane * 16;
#pragma unroll
          for (int kk = 0; kk < NKK; ++kk) {
            v8us zf[3];
#pragma unroll
            for (int t3 = 0; t3 < 3; ++t3) zf[t3] = *reinterpret_cast<const v8us*>(zb + (kk * 3 + t3) * kBlockBytes);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const v8bf bb = __builtin_bit_cast(
                  v8bf, *reinterpret_cast<const v8us*>(bb0 + ((size_t)j * NKK + kk) * kBlockBytes));
              v16f cur;
              if (kk == 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) cur[e] = 0.0f;
              } else {
                cur = lowS[j];
              }
              cur = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, zf[2]), bb, cur, 0, 0, 0);
              cur = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, zf[1]), bb, cur, 0, 0, 0);
              cur = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, zf[0]), bb, cur, 0, 0, 0);
              lowS[j] = cur;
            }
          }
          const float sgrp = g.lora_scaling[gi];
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) lowS[j][e] = lowS[j][e] * sgrp;
        }

        // ---- section B
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          // row 8*(v/4) + 4*h + v%4 of the block: its data sits in that lane (cross-lane read on
          // the LDS crossbar, which is idle here; no vector-ALU work)
          const int src_lane_addr = row_addr + 4 * (8 * (v >> 2) + (v & 3));
          const uint32_t rowoff = (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane_addr, (int)off_lane);
          const float sxv =
              __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane_addr, __builtin_bit_cast(int, sx_lane)));
          const float t0 = (float)acc[bi][2 * jp][v] * sxv;
          const float t1 = (float)acc[bi][2 * jp + 1][v] * sxv;
          // same f32 operations, in the same order, as the reference epilogue: a fused
          // multiply-add here would flip rare bf16 roundings that SwiGLU then amplifies
          float y0 = t0 * sw[2 * jp];
          float y1 = t1 * sw[2 * jp + 1];
          if constexpr (kLora) {
            y0 = y0 + lowS[0][v];
            y1 = y1 + lowS[1][v];
          }
          bool row_valid = fast || rowoff != 0xffffffffu;
          if (kLora && ghi > glo)  // boundary block: this pass owns only the rows of group gi
            row_valid = row_valid && (__builtin_amdgcn_ds_bpermute(src_lane_addr, grp_lane) == gi);
          uint32_t mine_bits;
          if (EPI == kEpiSwiglu) {
            // (y0, y1) = (gate, up) of the product column ncol/2 + jp
            const uint32_t f = pack_bf16x2(y0, y1);
            mine_bits = __float_as_uint(swiglu_f32(__uint_as_float(f << 16), __uint_as_float(f & 0xffff0000u)));
          } else {
            if (g.residual && row_valid) {
              uint32_t rr;
              if (fast) {
                rr = *reinterpret_cast<const uint32_t*>(g.residual + rowoff + ncol + 2u * jp);
              } else {
                rr = 0;
                if (ncol + 2u * jp < g.N) rr |= (uint32_t)g.residual[rowoff + ncol + 2u * jp];
                if (ncol + 2u * jp + 1u < g.N) rr |= (uint32_t)g.residual[rowoff + ncol + 2u * jp + 1u] << 16;
              }
              y0 = y0 + __uint_as_float(rr << 16);
              y1 = y1 + __uint_as_float(rr & 0xffff0000u);
            }
            mine_bits = pack_bf16x2(y0, y1);
          }
          if (jp == 0) {
            hold[v] = mine_bits;
            continue;
          }
          if (!row_valid) continue;
          if (EPI == kEpiSwiglu) {
            const uint32_t pk = pack_bf16x2(__uint_as_float(hold[v]), __uint_as_float(mine_bits));
            uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + rowoff + (ncol >> 1);
            if (fast) {
              *reinterpret_cast<uint32_t*>(o) = pk;
            } else {
              if ((ncol >> 1) < n_out) o[0] = (uint16_t)(pk & 0xffffu);
              if ((ncol >> 1) + 1u < n_out) o[1] = (uint16_t)(pk >> 16);
            }
          } else {
            uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + rowoff + ncol;
            if (fast) {
              *reinterpret_cast<uint2*>(o) = make_uint2(hold[v], mine_bits);
            } else {
              if (ncol + 0u < g.N) o[0] = (uint16_t)(hold[v] & 0xffffu);
              if (ncol + 1u < g.N) o[1] = (uint16_t)(hold[v] >> 16);
              if (ncol + 2u < g.N) o[2] = (uint16_t)(mine_bits & 0xffffu);
              if (ncol + 3u < g.N) o[3] = (uint16_t)(mine_bits >> 16);
            }
          }
        }
      }
      }  // groups of the block
    };
    epilogue_block(std::integral_constant<int, 0>{});
    if constexpr (kWR == 2) epilogue_block(std::integral_constant<int, 1>{});
  }
}

}  // namespace w8a8
