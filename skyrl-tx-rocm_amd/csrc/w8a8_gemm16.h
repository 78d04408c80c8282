// Tiled int8 GEMM with the fused float32 epilogue on 16 x 16 x 64 MFMAs:
//   acc[p, n]  = sum_k xq[p, k] * wq[k, n]                         (v_mfma_i32_16x16x64_i8, exact)
//   base       = (float(acc) * sx[p]) * sw[n]                      (skyrl/tx/kernels/quantized_lora.py:248-252)
//   y          = base + low * s[group(p)] (+ residual)             (quantized_lora.py:300-304)
//   low        = z[p, :] @ B[group(p)]                             (v_mfma_f32_16x16x32_bf16, z carried as 3 (or 2) bf16 terms)
//   out        = bf16(y)   or   bf16(silu(bf16(y_gate)) * bf16(y_up))
// Workgroup = 512 threads = 8 waves (2 x 4), tile 256 x 256, wave tile 128 x 64 = 8 x 4 blocks of
// 16 x 16: 128 accumulator registers per lane, two waves per SIMD, one workgroup per CU (a second
// wave on the SIMD fills the issue slots that LDS reads, waits, barriers and load issue cost the
// first; with one wave of 128 x 128 per SIMD the same loop ran at 1300 cycles per stage against the
// 1024 its MFMAs need).  K is consumed in steps of 64 through a ring of four 32 KiB LDS stages
// filled by 16-byte direct-to-LDS loads of contiguous 1 KiB fragment blocks, four steps ahead of
// the MFMAs; the ring runs on across tiles (the last four stages of a tile request the first four
// of the next), so the epilogue issues no stage loads and none of its own loads queues behind them.
// The 16 x 16 x 64 instruction is used because it moves a quarter of the accumulator bytes per
// operation of the 32 x 32 x 32 one: on random operands the part sustains about a fifth more
// operations per second with it before its power limit sets the clock.
//
// Operand mapping.  A 1 KiB fragment block holds 32 rows x 32 k; an MFMA operand is 16 rows x 64 k.
// Lane l (c16 = l % 16, q = l / 16) reads, from the two consecutive k blocks of a stage, its row
// c16 (+ 16 for the upper half of the block) in k block q / 2, k half q % 2: 16 consecutive lanes
// read 256 consecutive bytes, so the reads have no bank conflicts.  Activations are the A operand,
// weights the B operand: lane (c16, q) ends up with packed weight column c16 of a 16-column
// fragment and the four rows 4 q + v of a 16-row fragment.  With the column permutation of the
// packed weight (packed 32 j + c <-> original 4 c + j inside a group of 128) a wave takes, from
// each of the four 32-column blocks j of a group, the same half `chalf` of the columns: its four
// fragments give the lane the four consecutive original columns 4 (16 chalf + c16) + j of every
// one of its rows, and the wave 64 consecutive original columns.
//
// The direct-to-LDS loads are inline assembly with hand-counted s_waitcnt vmcnt in front of the
// barriers.  The compiler treats such a load as a FLAT access that may touch LDS and, while one is
// outstanding (here: always), turns every wait it inserts into vmcnt(0) / lgkmcnt(0); loads it does
// not know of can only make its own waits stricter, because the counters retire in order.  Nothing
// an assembly statement produces is a register value, so the compiler may spill and move freely.
#pragma once
#include <type_traits>

#include "w8a8_device.h"
#include "w8a8_gemm.h"

namespace w8a8 {

typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef uint32_t v2u_t __attribute__((ext_vector_type(2)));

constexpr int kG16TileM = 256;
constexpr int kG16TileN = 256;
constexpr uint32_t kG16MinKPad = 384;               // at least six stages: the schedule below assumes it
// Two geometries of the same kernel, told apart by NW, the waves side by side along N (2 rows of them):
//   NW = 4: tile 256 x 256, 8 waves, one workgroup per CU, ring of four 32 KiB stages;
//   NW = 2: tile 256 x 128, 4 waves, two independent workgroups per CU (one wave of each per SIMD), ring of
//           three 24 KiB stages each: while one workgroup runs its epilogue on the vector ALU the other's
//           main loop has the matrix core to itself.
// The wave tile (128 x 64), its fragment reads and its epilogue are the same in both.
template <int NW>
struct G16Geo {
  static constexpr int kTileN = 64 * NW;
  static constexpr int kStages = NW == 4 ? 4 : 3;
  static constexpr int kStageBytes = 16384 + 4096 * NW;  // A: 8 row blocks x 2 k blocks, then B: 2 NW column blocks x 2 k blocks
  static constexpr int kRingBytes = kStages * kStageBytes;
  static constexpr int kWaves = 2 * NW;
  static constexpr int kLdsBytes = kRingBytes + kWaves * 1024 + (NW == 4 ? 0 : 64);  // + per wave 128 row scales and 128 row positions (+ the next tile's position)
  static constexpr int kLoads = kStageBytes / 1024 / kWaves;     // direct-to-LDS loads per wave and stage (4 or 6)
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int kResident = NW == 4 ? 256 : 512;          // workgroups the chip holds at once
};
constexpr int kG16LdsBytes = G16Geo<4>::kLdsBytes;

// Four direct-to-LDS loads of 1 KiB each: lane l moves 16 bytes global[base_i + 1024 i + voff] -> LDS[lds_addr +
// 1024 i + 16 l] (voff = 16 l + ...).  The instruction offset applies to the global and to the LDS address
// alike, so the four loads share one M0 and the caller passes base_i = chunk address - 1024 i.
__device__ inline void g16_load_4k(const unsigned char* b0, const unsigned char* b1, const unsigned char* b2,
                                   const unsigned char* b3, uint32_t voff, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %5\n\ts_nop 0\n\t"
               "global_load_lds_dwordx4 %0, %1\n\t"
               "global_load_lds_dwordx4 %0, %2 offset:1024\n\t"
               "global_load_lds_dwordx4 %0, %3 offset:2048\n\t"
               "global_load_lds_dwordx4 %0, %4 offset:3072"
               :: "v"(voff), "s"(b0), "s"(b1), "s"(b2), "s"(b3), "s"(lds_addr_uniform) : "memory", "m0");
}
// Two more for the six-load geometry: chunks 4 and 5 of the wave, LDS address and global base 4 KiB on.
__device__ inline void g16_load_2k(const unsigned char* b4, const unsigned char* b5, uint32_t voff, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\t"
               "global_load_lds_dwordx4 %0, %1\n\t"
               "global_load_lds_dwordx4 %0, %2 offset:1024"
               :: "v"(voff), "s"(b4), "s"(b5), "s"(lds_addr_uniform) : "memory", "m0");
}
__device__ inline void g16_set_m0(uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" :: "s"(lds_addr_uniform) : "memory", "m0");
}
template <int OFF>
__device__ inline void g16_load_1k_m0(const unsigned char* base_uniform, uint32_t voff) {  // M0 set before
  asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" :: "v"(voff), "s"(base_uniform), "n"(OFF) : "memory", "m0");
}
// One wave copies 128 dwords: lane l moves global[base + 4 l] and global[base + 256 + 4 l] to the same
// offsets behind lds_addr.
__device__ inline void g16_load_128_dwords(const void* base_uniform, uint32_t lane4, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1\n\t"
               "global_load_lds_dword %0, %1 offset:256"
               :: "v"(lane4), "s"(base_uniform), "s"(lds_addr_uniform) : "memory", "m0");
}
// LDS fragment read.  These are ordinary loads the compiler keeps its books on: it places the waits
// (precisely, since it never sees the direct-to-LDS loads) and may spill or move the values safely.
template <int OFF>
__device__ inline v4i g16_ds_read(uint32_t addr) {
  typedef __attribute__((address_space(3))) const v4i* lds_v4i_ptr;
  return *reinterpret_cast<lds_v4i_ptr>((uintptr_t)(addr + OFF));
}
template <int N>
__device__ inline void g16_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }
template <int J0, int J1, class F>
__device__ inline void g16_for(F&& f) {  // f(integral_constant<int, J>) for J0 <= J < J1, unrolled at compile time
  if constexpr (J0 < J1) {
    f(std::integral_constant<int, J0>{});
    g16_for<J0 + 1, J1>(f);
  }
}
// The integer MFMAs are written as assembly with the accumulator tied (one read-write operand).  Through
// the builtin, destination and accumulator input are separate values, and in the stages ahead of and behind
// the steady-state loop the register allocator used that freedom: it placed 19 of a tile's 32 accumulator
// blocks elsewhere and moved them home through the vector registers, with the wait states that takes.
// What the compiler no longer sees is that an MFMA wrote the accumulator, so it inserts no wait states
// for a read of it by another unit; none is needed where this kernel reads one: a block is next touched by
// the MFMA of the following stage (32 MFMAs on), and the epilogue starts behind explicit wait states.
__device__ inline void g16_mfma(v4i& acc, const v4i& a, const v4i& b) {
  asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ inline void g16_mfma_first(v4i& acc, const v4i& a, const v4i& b) {
  asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}
constexpr int g16_frag_off(int f) { return (f >> 1) * 2048 + (f & 1) * 256; }  // activation fragment f of a wave's four row blocks
constexpr int g16_bfrag_off(int j) { return j * 2048; }                        // weight fragment j: the wave's half of column block j

template <int EPI, int NKK, int NW = 4>
__global__ __launch_bounds__(G16Geo<NW>::kThreads, NW == 4 ? 1 : 2)
void w8a8_gemm16_kernel(GemmArgs g) {
  using Geo = G16Geo<NW>;
  constexpr int kS = Geo::kStages;
  constexpr int kLoads = Geo::kLoads;
  constexpr uint32_t kSB = Geo::kStageBytes;
  auto ring = [](uint32_t i) -> uint32_t { return kS == 4 ? (i & 3u) : i % (uint32_t)kS; };
  constexpr bool kLora = (NKK > 0) && (EPI != kEpiAcc);
  constexpr int kKS = NKK > 2 ? 2 : 1;  // 32-wide rank steps of the LoRA product
  constexpr uint32_t kNkk = NKK > 0 ? NKK : 1;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wrow = wave / NW, wcol = wave % NW;  // wave tile: rows 128 wrow, columns 64 wcol of the tile
  const int cgrp = wcol >> 1, chalf = wcol & 1;  // its 128-column group inside the tile and its half of every block
  const uint32_t c16 = lane & 15, q = lane >> 4;
  // byte offset of the lane's 16 bytes inside a pair of k blocks (lower 16 rows of the block)
  const uint32_t lane_off = (q >> 1) * kBlockBytes + (c16 + 32u * (q & 1u)) * 16u;

  const uint32_t total_rows = g.total_rows;
  const uint32_t ntile = g.tiles_m * g.tiles_n;
  const uint32_t ncb_total = n_padded(g.N) / 32u;
  const uint32_t n_out = (EPI == kEpiSwiglu) ? g.N / 2u : g.N;
  const int KT = (int)(g.K_pad / 64u);  // even (K is padded to 128) and at least 6

  // ---- persistent schedule: consecutive workgroup ids land on different XCDs, so each XCD walks a
  // contiguous range of a band-major tile order (4 row tiles x all column tiles) and its workgroups
  // share panels in its own L2.
  const uint32_t per_xcd = (ntile + 7u) / 8u;
  const uint32_t wgs_per_xcd = gridDim.x >> 3;
  auto tile_at = [&](uint32_t i) -> GemmTile {
    GemmTile T{};
    const uint32_t t = i < per_xcd ? (blockIdx.x & 7u) * per_xcd + i : ntile;
    if (t >= ntile) return T;
    constexpr uint32_t GM = 4;
    const uint32_t band = t / (GM * g.tiles_n);
    const uint32_t band_rows = (g.tiles_m - band * GM) < GM ? (g.tiles_m - band * GM) : GM;
    const uint32_t in_band = t - band * GM * g.tiles_n;
    T.tm = band * GM + in_band % band_rows;
    T.tn = in_band / band_rows;
    T.Ag = g.xq + (size_t)T.tm * 8u * g.KB * kBlockBytes;
    T.Bg = g.wp;
    T.swp = g.sw;
    T.valid = true;
    return T;
  };
  // chunk ch = kLoads wave + i of a stage: 0..15 activations (row block ch / 2, k block ch % 2), 16..
  // weights; stage kt of a chunk lies 2 KiB * kt behind its base.  Returned: base - 1024 (i % 4), see
  // g16_load_4k.
  auto chunk_base = [&](const GemmTile& Tx, int i) -> const unsigned char* {
    const int ch = wave * kLoads + i;
    const bool isA = ch < 16;
    uint32_t rb = isA ? (uint32_t)(ch >> 1) : Tx.tn * (uint32_t)(2 * NW) + (uint32_t)((ch - 16) >> 1);
    if (!isA && rb >= ncb_total) rb = ncb_total - 1u;  // keep every wave's load count equal
    return (isA ? Tx.Ag : Tx.Bg) + ((size_t)rb * g.KB + (uint32_t)(ch & 1)) * kBlockBytes - (size_t)(i & 3) * 1024u;
  };
  // the wave's loads of one stage: lane offset voff inside the chunks, LDS address of its first chunk
  auto load_stage = [&](const unsigned char* const* cb, uint32_t voff, uint32_t dst) {
    if constexpr (kS != 4) dst = __builtin_amdgcn_readfirstlane(dst);  // (the ring position modulo 3 is formed on the vector ALU)
    g16_load_4k(cb[0], cb[1], cb[2], cb[3], voff, dst);
    if constexpr (kLoads == 6) g16_load_2k(cb[4], cb[5], voff, dst + 4096u);
  };

  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr_t)lds;
  const uint32_t a0 = lds_addr + (uint32_t)wrow * 8192u + lane_off;           // activation fragments, ring slot 0
  const uint32_t b0 = lds_addr + 16384u + (uint32_t)cgrp * 8192u + (uint32_t)chalf * 256u + lane_off;  // weight fragments, ring slot 0
  const uint32_t dma0 = lds_addr + (uint32_t)wave * (kLoads * kBlockBytes);  // the wave's chunks, ring slot 0
  // per wave: f32 sx[128] then int32 src_row[128] of its rows, behind the stage ring
  unsigned char* const rowdata = lds + Geo::kRingBytes + wave * 1024;  // (the waves of a row half hold the same data)

  // Raw buffer resources over the LoRA operands: loads through them take a uniform 64-bit base, a uniform
  // 32-bit offset and a 32-bit lane offset, so no lane holds a 64-bit address.
  const __amdgpu_buffer_rsrc_t zrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(g.zp), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t brsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(g.bp), 0, -1, 0x00020000);
  // The output through the same kind of resource, for fragments stored without conditions: a lane then
  // holds a 32-bit byte offset, which an output of less than 4 GiB (and 24-bit row and column counts,
  // for the one-instruction product) allows.
  const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(g.out, 0, -1, 0x00020000);
  const bool out_small = g.M < (1u << 24) && n_out < (1u << 24) && (uint64_t)g.M * n_out < (1ull << 31);
  uint32_t g0 = 0;          // ring slot of the current tile's stage 0
  bool prefetched = false;  // the first stages of the current tile were requested by the previous tile
  // Two workgroups per CU: the one the dispatcher placed first (its LDS allocation starts at 0) runs at a
  // higher wave priority.  Its main loop then takes every matrix-core slot it can use and the other
  // workgroup fills the rest -- all of them while the first is in its epilogue -- instead of both running
  // their main loops and then their epilogues side by side.  Positions beyond the first come from the
  // XCD's counter, since the two no longer finish their tiles at the same rate.
  constexpr bool kDyn = NW != 4;
  uint32_t* const next_slot = reinterpret_cast<uint32_t*>(lds + Geo::kRingBytes + Geo::kWaves * 1024);
  uint32_t* const ctr = g.tile_ctr + (blockIdx.x & 7u) * 16u;
  uint32_t cur_i = blockIdx.x >> 3, nxt_i = cur_i + wgs_per_xcd;
  if constexpr (kDyn) {
    uint32_t lds_alloc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_LDS_ALLOC, 0, 8)" : "=s"(lds_alloc));
    if (lds_alloc == 0u) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(0);
    if (tid == 0) *next_slot = wgs_per_xcd + atomicAdd(ctr, 1u);
    __syncthreads();
  }
  auto advance = [&]() {
    cur_i = nxt_i;
    if constexpr (!kDyn) nxt_i = cur_i + wgs_per_xcd;
  };
  for (; cur_i < per_xcd; advance()) {
    const GemmTile T = tile_at(cur_i);
    if (!T.valid) break;  // positions only grow: nothing valid follows

    const unsigned char* cbase[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) cbase[i] = chunk_base(T, i);

    v4i acc[8][4];
    v4i bf[2][4];  // weight fragments of the current / next stage
    v4i af[4];     // activation fragments, three ahead of the MFMAs
    if (!prefetched) {
#pragma unroll
      for (int st = 0; st < kS; ++st) {
        const uint32_t voff = (uint32_t)st * 2048u + (uint32_t)lane * 16u;
        const uint32_t dst = dma0 + ring((uint32_t)st + g0) * kSB;
        load_stage(cbase, voff, dst);
      }
    }
    // Stage 0 must have landed.  Behind it in the queue: the other stages of the ring and, when the previous
    // tile requested them, that tile's epilogue, which is younger still.
    g16_wait_vm<(kS - 1) * kLoads>();
    lds_barrier();
    if constexpr (kDyn) nxt_i = __builtin_amdgcn_readfirstlane(*reinterpret_cast<volatile uint32_t*>(next_slot));
    GemmTile Tn{};
    if (nxt_i < per_xcd) Tn = tile_at(nxt_i);
    const bool has_next = Tn.valid;  // workgroup-uniform

    // LDS reads retire in order; the waits below count the reads issued behind the one they need.
    // Order here and at the end of every stage: B0..B3, A0, A1, A2.
    {
      const uint32_t sa = a0 + ring(g0) * kSB, sb = b0 + ring(g0) * kSB;
      g16_for<0, 4>([&](auto J) { bf[0][decltype(J)::value] = g16_ds_read<g16_bfrag_off(decltype(J)::value)>(sb); });
      af[0] = g16_ds_read<g16_frag_off(0)>(sa);
      af[1] = g16_ds_read<g16_frag_off(1)>(sa);
      af[2] = g16_ds_read<g16_frag_off(2)>(sa);
    }

    const unsigned char* nbase[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) nbase[i] = has_next ? chunk_base(Tn, i) : cbase[i];

    // One stage: 32 MFMAs per wave.  Activation fragment bi + 3 is fetched under the MFMAs of fragment
    // bi; before fragment 6 the next stage must have landed (own loads counted, then the barrier), the
    // buffer of this stage is handed to the loads four stages ahead, and the next stage's first
    // fragments are fetched under the last 8 MFMAs.  REM = stages of this tile after this one, capped
    // at 4: a compile-time constant, so that the steady-state loop body has no branches.  With REM < 4
    // the stage four ahead belongs to the next tile.
    auto stage = [&](auto PAR, auto FIRST, auto REMC, int kt) {
      constexpr int P = decltype(PAR)::value;
      constexpr bool first = decltype(FIRST)::value;
      constexpr int REM = decltype(REMC)::value;
      // The stage addresses are formed from values the compiler cannot see through: it would otherwise
      // compute every stage's addresses once at kernel start and keep them in registers (or spill them).
      uint32_t a0s = a0, b0s = b0;
      asm volatile("" : "+v"(a0s), "+v"(b0s));
      const uint32_t slot = ring((uint32_t)kt + g0), slot_n = ring((uint32_t)kt + 1u + g0);
      const uint32_t sa = a0s + slot * kSB;
      const uint32_t san = a0s + slot_n * kSB;
      const uint32_t sbn = b0s + slot_n * kSB;
      auto mfma_row = [&](auto BI) {
        constexpr int bi = decltype(BI)::value;
#pragma unroll
        for (int bj = 0; bj < 4; ++bj) {
          if constexpr (first) g16_mfma_first(acc[bi][bj], af[bi & 3], bf[P][bj]);
          else g16_mfma(acc[bi][bj], af[bi & 3], bf[P][bj]);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      using std::integral_constant;
      // in flight here, oldest first: B0..B3, A0, A1, A2 of this stage
      af[3] = g16_ds_read<g16_frag_off(3)>(sa);
      mfma_row(integral_constant<int, 0>{});
      af[0] = g16_ds_read<g16_frag_off(4)>(sa);
      mfma_row(integral_constant<int, 1>{});
      af[1] = g16_ds_read<g16_frag_off(5)>(sa);
      mfma_row(integral_constant<int, 2>{});
      af[2] = g16_ds_read<g16_frag_off(6)>(sa);
      mfma_row(integral_constant<int, 3>{});
      af[3] = g16_ds_read<g16_frag_off(7)>(sa);
      mfma_row(integral_constant<int, 4>{});
      mfma_row(integral_constant<int, 5>{});
      // The next stage must have landed: own loads first, then everybody's; the barrier also ends every
      // wave's reads of this stage's buffer.  Three stages are in the queue behind this one as long as
      // the tile or a next tile provides them.
      if constexpr (REM >= kS - 1) {
        g16_wait_vm<(kS - 2) * kLoads>();
      } else if constexpr (REM >= 1) {
        if (has_next) g16_wait_vm<(kS - 2) * kLoads>();
        else g16_wait_vm<(REM - 1) * kLoads>();
      }
      lds_barrier();  // REM == 0: nothing has to land here; the barrier frees this stage's buffer
      // After the barrier the last 8 MFMAs start at once (their operands are in registers); the next
      // stage's first fragments (order B0..B3, A0, A1, A2) and the four loads of the stage four ahead
      // (into the buffer the barrier has just freed) are issued in the gaps between them.  The order is
      // pinned: bunched in front of the MFMAs, these ten instructions per wave leave the matrix core idle.
      auto one = [&](auto BI, auto BJ) {
        constexpr int bi = decltype(BI)::value, bj = decltype(BJ)::value;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (first) g16_mfma_first(acc[bi][bj], af[bi & 3], bf[P][bj]);
        else g16_mfma(acc[bi][bj], af[bi & 3], bf[P][bj]);
        __builtin_amdgcn_sched_barrier(0);
      };
      using C6 = integral_constant<int, 6>;
      using C7 = integral_constant<int, 7>;
      one(C6{}, integral_constant<int, 0>{});
      if constexpr (REM >= 1) {
        bf[1 - P][0] = g16_ds_read<g16_bfrag_off(0)>(sbn);
        bf[1 - P][1] = g16_ds_read<g16_bfrag_off(1)>(sbn);
      }
      one(C6{}, integral_constant<int, 1>{});
      if constexpr (REM >= 1) {
        bf[1 - P][2] = g16_ds_read<g16_bfrag_off(2)>(sbn);
        bf[1 - P][3] = g16_ds_read<g16_bfrag_off(3)>(sbn);
      }
      one(C6{}, integral_constant<int, 2>{});
      if constexpr (REM >= 1) {
        af[0] = g16_ds_read<g16_frag_off(0)>(san);
        af[1] = g16_ds_read<g16_frag_off(1)>(san);
      }
      one(C6{}, integral_constant<int, 3>{});
      one(C7{}, integral_constant<int, 0>{});
      if constexpr (REM >= 1) af[2] = g16_ds_read<g16_frag_off(2)>(san);
      if (REM >= kS || (REM >= 1 && has_next)) {  // compile-time facts but has_next; the last stage issues none
        const uint32_t voff4 = (uint32_t)(REM >= kS ? kt + kS : kt + kS - KT) * 2048u + (uint32_t)lane * 16u;
        if constexpr (REM >= kS) load_stage(cbase, voff4, dma0 + slot * kSB);
        else load_stage(nbase, voff4, dma0 + slot * kSB);
      }
      one(C7{}, integral_constant<int, 1>{});
      one(C7{}, integral_constant<int, 2>{});
      one(C7{}, integral_constant<int, 3>{});
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>;
    using Yes = std::true_type;
    using No = std::false_type;
    stage(I0{}, Yes{}, I4{}, 0);
    stage(I1{}, No{}, I4{}, 1);
    for (int kt = 2; kt < KT - 4; kt += 2) {
      stage(I0{}, No{}, I4{}, kt);
      stage(I1{}, No{}, I4{}, kt + 1);
    }
    stage(I0{}, No{}, I3{}, KT - 4);
    stage(I1{}, No{}, I2{}, KT - 3);
    stage(I0{}, No{}, I1{}, KT - 2);
    // adapters present in the wave's four 32-row blocks: one scalar load (the compiler would
    // fetch them through the vector memory path and wait vmcnt(0))
    v4i range4 = {0, 0, 0, 0};
    if (kLora && g.blk_range)
      asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)"
                   : "=s"(range4) : "s"(g.blk_range + (T.tm * 256u + wrow * 128u) / 32u) : "memory");
    // ---- What the epilogue works with is set up here, behind the main loop's bulk, so that none of it
    // is live (or spilled) across the loop; preload() requests what it starts from.
    const uint32_t m0 = T.tm * 256u + wrow * 128u;     // first slot of the wave
    const uint32_t tgrp0 = T.tn * (uint32_t)Geo::kTileN + cgrp * 128u;  // first column of the wave's group of 128
    const uint32_t tcol0 = tgrp0 + chalf * 64u;        // first of the wave's 64 columns
    const bool wave_live = tcol0 < g.N;                // wave-uniform; a dead wave only feeds the loads
    const bool full_n = (tcol0 + 64u <= g.N) && ((g.N & 3u) == 0);  // wave-uniform
    const v4i zero4 = {0, 0, 0, 0};
    v4i swr = zero4;                                   // per-channel scales of the lane's 4 columns
    const uint32_t range[4] = {(uint32_t)range4.x, (uint32_t)range4.y, (uint32_t)range4.z, (uint32_t)range4.w};
    v4i zr[2][kKS][3];                                 // z operands: ring of two 16-row fragments
    v4i br[4][kKS];                                    // LoRA B operands of adapter `bgroup`
    // (defined on every path: an undefined start would let the last tile's values count as live across the loop)
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
#pragma unroll
      for (int t3 = 0; t3 < 3; ++t3) zr[0][ks][t3] = zr[1][ks][t3] = zero4;
#pragma unroll
      for (int bj = 0; bj < 4; ++bj) br[bj][ks] = zero4;
    }
    int bgroup = -1;
    float bscale = 0.0f;  // lora_scaling[bgroup]
    // operand bytes inside a 1 KiB block of the 32 x 16 layouts the prologue writes: rank octet q sits in
    // rank chunk q / 2 (16 ranks each), half q % 2.  A rank chunk beyond the rank is read from the last
    // existing one and zeroed afterwards.
    uint32_t lora_lane = (c16 + 32u * (q & 1u)) * 16u;
    asm volatile("" : "+v"(lora_lane));  // per tile: keeps the derived lane offsets out of kernel-long registers
    const bool lane_has_rank[2] = {(q >> 1) < kNkk, 2u + (q >> 1) < kNkk};
    // z and B are read through buffer resources: a uniform offset per operand and, per 32-rank step,
    // one lane offset (rank chunk of the lane, clamped to the last existing one, and lane position).
    uint32_t zlane[kKS], blane[kKS];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
      uint32_t kk = 2u * ks + (q >> 1);
      if (kk >= kNkk) kk = kNkk - 1u;
      zlane[ks] = kk * 3u * kBlockBytes + lora_lane;
      blane[ks] = kk * kBlockBytes + lora_lane;
    }
    auto z_soff = [&](int bi, int t3) -> uint32_t {
      return ((m0 / 32u + (uint32_t)(bi >> 1)) * kNkk * 3u + (uint32_t)t3) * kBlockBytes + (uint32_t)(bi & 1) * 256u;
    };
    auto b_soff = [&](int gi, int bj) -> uint32_t {
      return (((uint32_t)gi * ncb_total + tgrp0 / 32u + (uint32_t)bj) * kNkk) * kBlockBytes + (uint32_t)chalf * 256u;
    };
    auto load_z = [&](int slot, int bi) {
#pragma unroll
      for (int ks = 0; ks < kKS; ++ks)
#pragma unroll
        for (int t3 = 0; t3 < 3; ++t3)
          zr[slot][ks][t3] = lane_has_rank[ks] ? __builtin_amdgcn_raw_buffer_load_b128(zrsrc, zlane[ks], z_soff(bi, t3), 0) : zero4;
    };
    auto load_b = [&](int gi) {
#pragma unroll
      for (int bj = 0; bj < 4; ++bj)
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks)
          br[bj][ks] = lane_has_rank[ks] ? __builtin_amdgcn_raw_buffer_load_b128(brsrc, blane[ks], b_soff(gi, bj), 0) : zero4;
      bgroup = gi;
      // the adapter's scaling through the scalar path, once per adapter: a vector load at its use would be
      // waited for with vmcnt(0), behind the operand loads of the fragments to come and the next tile's stage
      asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(bscale) : "s"(g.lora_scaling + gi) : "memory");
    };
    // What the epilogue starts from is requested at the start of the last stage, with loads the compiler
    // keeps its books on (it places the waits and may move the values as it likes).  No stage load is
    // issued behind them before they are waited for, so that wait does not stall on a younger load.
    uint32_t grabbed = 0;  // the position after next of a dynamic schedule, requested with the epilogue's operands
    auto preload = [&]() {
      if (kDyn && tid == 0) grabbed = atomicAdd(ctr, 1u);
      if (EPI != kEpiAcc) g16_load_128_dwords(g.sx + m0, (uint32_t)lane * 4u, lds_addr + Geo::kRingBytes + wave * 1024);
      if (g.src_row) g16_load_128_dwords(g.src_row + m0, (uint32_t)lane * 4u, lds_addr + Geo::kRingBytes + wave * 1024 + 512);
      if (!wave_live) return;
      if (EPI != kEpiAcc && full_n) swr = *reinterpret_cast<const v4i*>(T.swp + tcol0 + 4u * c16);
      if constexpr (kLora) {
        load_z(0, 0);  // (the second fragment's operands are requested when the epilogue starts: during the
                       // last stage their twelve registers are still needed for its operands)
        load_b((int)(range[0] & 0xffffu));
      }
    };

    preload();
    stage(I1{}, No{}, I0{}, KT - 1);  // the last stage (KT is even); it also requests the epilogue's operands
    // (wait states between the last MFMAs and whatever the compiler schedules next: it does not know that the
    // accumulators were just written, see g16_mfma; sixteen cover this MFMA's result latency)
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
    // The preloads were requested a stage ago and are the youngest loads in the queue.  After the wait
    // (the builtin, so that the compiler knows its loads are in) the next tile's fourth stage is requested
    // into the buffer the last barrier has freed.
    wait_vmcnt<0>();
    if (kDyn && tid == 0) *next_slot = wgs_per_xcd + grabbed;  // read by every wave behind the next tile's first barrier
    if (has_next) {
      const uint32_t voff = (uint32_t)(kS - 1) * 2048u + (uint32_t)lane * 16u;
      load_stage(nbase, voff, dma0 + ring((uint32_t)KT - 1u + g0) * kSB);
    }
    g0 = ring(g0 + (uint32_t)KT);
    prefetched = has_next;

    // ---------------------------------------------------------------- epilogue
    // Lane (c16, q) owns, in every 16-row fragment bi, the rows 4 q + v (v = 0..3) and the four
    // consecutive original columns tcol0 + 4 c16 + j held by the accumulator blocks j.
    if (!wave_live) continue;  // wave beyond the last column; it still takes part in the next tile
    if constexpr (kLora) load_z(1, 1);
    // Does every one of the wave's 128 slots hold a row of the output, and every lane four columns?
    // (wave-uniform; true for all but the tiles at the end of an adapter's rows or of the matrix)
    bool tile_plain = out_small && full_n && m0 + 128u <= total_rows;
    if (g.src_row) {
      const int2 s2 = *reinterpret_cast<const int2*>(rowdata + 512u + (uint32_t)lane * 8u);
      const bool both = (uint32_t)s2.x < g.M && (uint32_t)s2.y < g.M;
      tile_plain = tile_plain && (__builtin_amdgcn_ballot_w64(!both) == 0);
    } else {
      tile_plain = tile_plain && m0 + 128u <= g.M;
    }
    const uint32_t ncol = tcol0 + 4u * c16;  // the lane's four consecutive columns
    float sw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sw[j] = full_n ? __int_as_float(swr[j]) : 0.0f;  // (a bit_cast of a vector element reads element 0)
    if (EPI != kEpiAcc && !full_n) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (ncol + j < g.N) sw[j] = T.swp[ncol + j];
    }
    g16_for<0, 8>([&](auto BI) {
      constexpr int bi = decltype(BI)::value;
      const uint32_t pbase = m0 + bi * 16u;  // first slot of the 16-row fragment
      if (pbase >= total_rows) return;       // wave-uniform
      __builtin_amdgcn_sched_barrier(0);     // keep the fragments' register lifetimes apart
      // the fragment's accumulators leave the accumulation registers here, not earlier
      asm volatile("" : "+a"(acc[bi][0]), "+a"(acc[bi][1]), "+a"(acc[bi][2]), "+a"(acc[bi][3]));
      const uint32_t p4 = pbase + 4u * q;
      float sx[4] = {0.f, 0.f, 0.f, 0.f};
      if (EPI != kEpiAcc) {
        const float4 s4 = *reinterpret_cast<const float4*>(rowdata + (16u * bi + 4u * q) * 4u);
        sx[0] = s4.x; sx[1] = s4.y; sx[2] = s4.z; sx[3] = s4.w;
      }
      int src[4] = {(int)p4, (int)p4 + 1, (int)p4 + 2, (int)p4 + 3};
      if (g.src_row) {
        const int4 r4 = *reinterpret_cast<const int4*>(rowdata + 512u + (16u * bi + 4u * q) * 4u);
        src[0] = r4.x; src[1] = r4.y; src[2] = r4.z; src[3] = r4.w;
      }
      // Groups (adapters) present in the 32-row block of this fragment: one, except at a group
      // boundary.  A boundary fragment is processed once per group; each pass stores its own rows.
      const int glo = (int)(range[bi >> 1] & 0xffffu), ghi = (int)(range[bi >> 1] >> 16);
      // The plain fragment (wave-uniform): every row of the wave's tile exists and all four columns of every
      // lane exist.  It runs without per-row conditions and stores through the buffer path; where two
      // adapters meet in its 32-row block, each adapter's pass stores the rows that are its own.
      const bool plain = EPI != kEpiAcc && tile_plain;
      const bool boundary = kLora && ghi > glo;
      bool row_ok[4] = {true, true, true, true};
      uint32_t off[4];
      bool fast = true;
      if (plain) {
#pragma unroll
        for (int v = 0; v < 4; ++v) off[v] = __umul24((uint32_t)src[v], n_out);
      } else {
        bool all_ok = true;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          row_ok[v] = src[v] >= 0 && src[v] < (int)g.M;
          off[v] = row_ok[v] ? (uint32_t)src[v] * ((EPI == kEpiAcc) ? g.N : n_out) : 0u;
          all_ok = all_ok && row_ok[v];
        }
        fast = full_n && (__builtin_amdgcn_ballot_w64(!all_ok) == 0);  // wave-uniform
      }

      if constexpr (EPI == kEpiAcc) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          if (!row_ok[v]) continue;
          int32_t* o = reinterpret_cast<int32_t*>(g.out) + off[v] + ncol;
          if (fast) {
            *reinterpret_cast<int4*>(o) = make_int4(acc[bi][0][v], acc[bi][1][v], acc[bi][2][v], acc[bi][3][v]);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (ncol + j < g.N) o[j] = acc[bi][j][v];
          }
        }
      } else {
        int grp[4] = {glo, glo, glo, glo};
        if (kLora && g.slot_group && ghi > glo) {
          const int4 g4 = *reinterpret_cast<const int4*>(g.slot_group + p4);
          grp[0] = g4.x; grp[1] = g4.y; grp[2] = g4.z; grp[3] = g4.w;
        }
        for (int gi = glo; gi <= ghi; ++gi) {  // wave-uniform (one pass, except at a boundary)
          // ---- low[bj][v] = s_g * (z @ B_g): z rows of this fragment, B columns of fragment bj.  The
          // three terms of a fragment run as three rounds over the four independent accumulators.
          v4f_t low[4];
          if constexpr (kLora) {
            if (gi != bgroup) load_b(gi);  // wave-uniform: a new adapter begins in this fragment
            const float sgrp = bscale;
            // The low-rank accumulators live in ordinary registers (every accumulation register is taken by the
            // integer accumulators), and the MFMAs write them there: assembly with the accumulator tied, as
            // g16_mfma.  An accumulator's next MFMA is four MFMAs on; the wait states between the last MFMA
            // and the first read by the vector ALU, which the compiler would insert for a builtin, are explicit.
#pragma unroll
            for (int ks = 0; ks < kKS; ++ks)
#pragma unroll
              for (int t3 = 2; t3 >= 0; --t3)
#pragma unroll
                for (int bj = 0; bj < 4; ++bj) {
                  if (ks == 0 && t3 == 2)  // (folded once the loops are unrolled)
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=&v"(low[bj]) : "v"(zr[bi & 1][ks][t3]), "v"(br[bj][ks]));
                  else
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(low[bj]) : "v"(zr[bi & 1][ks][t3]), "v"(br[bj][ks]));
                }
            asm volatile("s_nop 7\n\ts_nop 7" : "+v"(low[0]), "+v"(low[1]), "+v"(low[2]), "+v"(low[3]));
            if (sgrp != 1.0f) {  // wave-uniform (a product with 1 is exact: leaving it out changes no bit)
#pragma unroll
              for (int bj = 0; bj < 4; ++bj)
#pragma unroll
                for (int v = 0; v < 4; ++v) low[bj][v] = low[bj][v] * sgrp;
            }
          }
          // the fragment's rows; MODE 0 is the general form, 1 the plain one, 2 the plain one of a boundary pass
          auto rows = [&](auto MODE) {
            constexpr bool kPlain = decltype(MODE)::value != 0;
            constexpr bool kOwnRows = decltype(MODE)::value == 2;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              bool row_valid = true;
              uint32_t offv = off[v], ncolv = ncol;
              if constexpr (!kPlain) {
                row_valid = row_ok[v];
                if (kLora && ghi > glo) row_valid = row_valid && (grp[v] == gi);  // boundary: own rows only
                // (the addresses and column conditions of this form are formed here, not ahead of the branch
                // where the plain form would pay for them too)
                asm volatile("" : "+v"(offv), "+v"(ncolv));
              }
              float y[4];
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                // same f32 operations, in the same order, as the reference epilogue: a fused
                // multiply-add here would flip rare bf16 roundings that SwiGLU then amplifies
                const float t = (float)acc[bi][j][v] * sx[v];
                y[j] = t * sw[j];
                if constexpr (kLora) y[j] = y[j] + low[j][v];
              }
              if (EPI == kEpiSwiglu) {
                // (y0, y1) and (y2, y3) are the (gate, up) pairs of product columns ncol/2, ncol/2 + 1
                const uint32_t f0 = pack_bf16x2(y[0], y[1]), f1 = pack_bf16x2(y[2], y[3]);
                const float p0 = swiglu_f32(__uint_as_float(f0 << 16), __uint_as_float(f0 & 0xffff0000u));
                const float p1 = swiglu_f32(__uint_as_float(f1 << 16), __uint_as_float(f1 & 0xffff0000u));
                if (!kPlain && !row_valid) continue;
                const uint32_t pk = pack_bf16x2(p0, p1);
                if constexpr (kPlain) {
                  if (!kOwnRows || grp[v] == gi) __builtin_amdgcn_raw_buffer_store_b32(pk, orsrc, 2u * offv + ncolv, 0, 0);
                } else {
                  uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + offv + (ncolv >> 1);
                  if (fast) {
                    *reinterpret_cast<uint32_t*>(o) = pk;
                  } else {
                    if ((ncolv >> 1) < n_out) o[0] = (uint16_t)(pk & 0xffffu);
                    if ((ncolv >> 1) + 1u < n_out) o[1] = (uint16_t)(pk >> 16);
                  }
                }
              } else {
                if (!kPlain && !row_valid) continue;
                if (g.residual) {
                  uint32_t r0 = 0, r1 = 0;
                  if (kPlain || fast) {
                    const uint2 rr = *reinterpret_cast<const uint2*>(g.residual + offv + ncolv);
                    r0 = rr.x; r1 = rr.y;
                  } else {
                    if (ncolv + 0u < g.N) r0 |= (uint32_t)g.residual[offv + ncolv + 0u];
                    if (ncolv + 1u < g.N) r0 |= (uint32_t)g.residual[offv + ncolv + 1u] << 16;
                    if (ncolv + 2u < g.N) r1 |= (uint32_t)g.residual[offv + ncolv + 2u];
                    if (ncolv + 3u < g.N) r1 |= (uint32_t)g.residual[offv + ncolv + 3u] << 16;
                  }
                  y[0] = y[0] + __uint_as_float(r0 << 16);
                  y[1] = y[1] + __uint_as_float(r0 & 0xffff0000u);
                  y[2] = y[2] + __uint_as_float(r1 << 16);
                  y[3] = y[3] + __uint_as_float(r1 & 0xffff0000u);
                }
                const uint32_t lo = pack_bf16x2(y[0], y[1]), hi = pack_bf16x2(y[2], y[3]);
                if constexpr (kPlain) {
                  if (!kOwnRows || grp[v] == gi) __builtin_amdgcn_raw_buffer_store_b64(v2u_t{lo, hi}, orsrc, 2u * (offv + ncolv), 0, 0);
                } else {
                  uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + offv + ncolv;
                  if (fast) {
                    *reinterpret_cast<uint2*>(o) = make_uint2(lo, hi);
                  } else {
                    if (ncolv + 0u < g.N) o[0] = (uint16_t)(lo & 0xffffu);
                    if (ncolv + 1u < g.N) o[1] = (uint16_t)(lo >> 16);
                    if (ncolv + 2u < g.N) o[2] = (uint16_t)(hi & 0xffffu);
                    if (ncolv + 3u < g.N) o[3] = (uint16_t)(hi >> 16);
                  }
                }
              }
            }
          };
          if (!plain) rows(std::integral_constant<int, 0>{});
          else if (!boundary) rows(std::integral_constant<int, 1>{});
          else rows(std::integral_constant<int, 2>{});
        }  // groups of the fragment
        // this fragment's z operands are spent: their ring slot takes the fragment two ahead
        if constexpr (kLora && bi + 2 < 8) load_z(bi & 1, bi + 2);
      }
    });
  }
}

}  // namespace w8a8
