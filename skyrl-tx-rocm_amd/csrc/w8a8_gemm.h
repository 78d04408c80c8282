// Tiled int8 MFMA GEMM with the fused float32 epilogue:
//   acc[p, n]  = sum_k xq[p, k] * wq[k, n]                         (v_mfma_i32_32x32x32_i8, exact)
//   base       = (float(acc) * sx[p]) * sw[n]                      (skyrl/tx/kernels/quantized_lora.py:248-252)
//   y          = base + low * s[group(p)] (+ residual)             (quantized_lora.py:300-304)
//   low        = z[p, :] @ B[group(p)]                             (bf16 MFMA, z carried as 2-3 bf16 terms)
//   out        = bf16(y)   or   bf16(silu(bf16(y_gate)) * bf16(y_up))
// Workgroup = 256 threads = 4 waves, tile 256 x 256, K step 128, two LDS stages of 64 KiB
// filled by 16-byte direct-to-LDS loads of contiguous 1 KiB fragment blocks.
#pragma once
#include <type_traits>

#include "w8a8_device.h"

namespace w8a8 {

enum { kEpiPlain = 0, kEpiSwiglu = 1, kEpiAcc = 2 };

struct GemmArgs {
  const unsigned char* xq;   // packed activation codes [slots, K_pad]
  const unsigned char* wp;   // packed weight [N_pad, K_pad] (per group: + group * w_group_stride)
  const float* sx;           // f32 [slots]
  const float* sw;           // f32 [N] (per group: + group * N)
  const float* z_part;       // f32 [ksplit, slots, r_pad] or null
  const uint16_t* lora_b;    // bf16 [n_groups, rank, N] or null
  const float* lora_scaling; // f32 [n_groups]
  const int32_t* src_row;    // or null
  const int32_t* blk_group;  // or null
  const int32_t* meta;       // or null
  const uint16_t* residual;  // bf16 [M, n_out] or null
  void* out;                 // bf16 [M, n_out] or int32 [M, N]
  uint64_t w_group_stride;   // bytes between per-group packed weights (0 = shared weight)
  uint32_t M, N, K_pad, KB, slots, rows_static;
  uint32_t tiles_m, tiles_n, rank, r_pad, ksplit, nsplit_terms, grouped;
};

template <int EPI>
__global__ __launch_bounds__(256, 1) void w8a8_gemm_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // ---- XCD-aware tile mapping: consecutive workgroup ids land on different XCDs, so each
  // XCD gets a contiguous range of a band-major tile order (4 row tiles x all column tiles).
  const uint32_t total_rows = g.meta ? (uint32_t)g.meta[0] : g.rows_static;
  const uint32_t ntile = g.tiles_m * g.tiles_n;
  const uint32_t per_xcd = (ntile + 7u) / 8u;
  const uint32_t t = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
  if (t >= ntile) return;
  constexpr uint32_t GM = 4;
  const uint32_t band = t / (GM * g.tiles_n);
  const uint32_t band_rows = (g.tiles_m - band * GM) < GM ? (g.tiles_m - band * GM) : GM;
  const uint32_t in_band = t - band * GM * g.tiles_n;
  const uint32_t tm = band * GM + in_band % band_rows;
  const uint32_t tn = in_band / band_rows;
  if (tm * 256u >= total_rows) return;

  // grouped (ragged) mode: a whole row tile may span several groups; weights are per group,
  // so a tile is processed once per 32-row block run with one weight.  To keep the main loop
  // simple the grouped launcher guarantees one group per row tile (tile rows = 32-row blocks
  // of a single group); see launch code.  Dense mode shares one weight.
  const uint32_t tile_group = (g.grouped && g.blk_group) ? (uint32_t)g.blk_group[tm * 8u] : 0u;

  const unsigned char* Ag = g.xq + (size_t)tm * 8u * g.KB * kBlockBytes;
  const unsigned char* Bg = g.wp + (size_t)tile_group * g.w_group_stride + (size_t)tn * 8u * g.KB * kBlockBytes;
  const float* swg = g.sw + (size_t)tile_group * (g.grouped ? g.N : 0u);

  v16i acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  const int KT = (int)(g.K_pad / kTileK);
  auto issue = [&](int kt, int stage) {
    unsigned char* As = lds + stage * 65536;
    unsigned char* Bs = As + 32768;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int c = wave * 8 + q;  // chunk: row block c / 4 (0..7), k block c % 4
      const size_t goff = ((size_t)(c >> 2) * g.KB + (size_t)kt * 4 + (c & 3)) * kBlockBytes + lane * 16;
      load_1k_to_lds(Ag + goff, As + c * kBlockBytes);
      load_1k_to_lds(Bg + goff, Bs + c * kBlockBytes);
    }
  };

  issue(0, 0);
  wait_vmcnt0();
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    if (kt + 1 < KT) issue(kt + 1, (kt + 1) & 1);
    const unsigned char* As = lds + (kt & 1) * 65536;
    const unsigned char* Bs = As + 32768;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      v4i af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        af[i] = *reinterpret_cast<const v4i*>(As + ((wm * 4 + i) * 4 + ks) * kBlockBytes + lane * 16);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        bf[j] = *reinterpret_cast<const v4i*>(Bs + ((wn * 4 + j) * 4 + ks) * kBlockBytes + lane * 16);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    wait_vmcnt0();
    __syncthreads();
  }

  // ------------------------------------------------------------------ epilogue
  const int c = lane & 31, h = lane >> 5;
  const uint32_t m0 = tm * 256u + wm * 128u;           // first grouped slot of this wave
  const uint32_t n0 = tn * 256u + wn * 128u;           // first packed column of this wave
  const uint32_t n_out = (EPI == kEpiSwiglu) ? g.N / 2u : g.N;
  // LoRA-B staging, one buffer per wave row (wm): bf16 [r_pad][256] at lds + wm * 32 KiB
  uint16_t* Bl = reinterpret_cast<uint16_t*>(lds + wm * 32768);
  int staged0 = -1, staged1 = -1;
  const bool has_lora = (EPI != kEpiAcc) && g.r_pad > 0 && g.z_part != nullptr;

  auto epilogue_block = [&](auto BI) {
    constexpr int bi = decltype(BI)::value;
    const uint32_t blk0 = tm * 8u + bi, blk1 = blk0 + 4u;
    const bool act0 = blk0 * 32u < total_rows, act1 = blk1 * 32u < total_rows;
    const int grp0 = act0 ? (g.blk_group ? g.blk_group[blk0] : 0) : staged0;
    const int grp1 = act1 ? (g.blk_group ? g.blk_group[blk1] : 0) : staged1;
    const bool active = wm ? act1 : act0;
    const int grp = wm ? grp1 : grp0;
    if (has_lora && (grp0 != staged0 || grp1 != staged1)) {  // uniform over the workgroup
      __syncthreads();
      const int mine = wm ? staged1 : staged0;
      if (grp != mine && grp >= 0) {
        const uint16_t* Bsrc = g.lora_b + (size_t)grp * g.rank * g.N;
        const uint32_t ncol0 = tn * 256u;
        const uint32_t t128 = (uint32_t)(tid & 127);
        for (uint32_t q = t128; q < g.r_pad * 32u; q += 128) {
          const uint32_t r = q >> 5, cc = (q & 31u) * 8u;
          v8us val = {0, 0, 0, 0, 0, 0, 0, 0};
          if (r < g.rank) {
            const size_t off = (size_t)r * g.N + ncol0 + cc;
            if ((g.N & 7u) == 0 && ncol0 + cc + 8u <= g.N) {
              val = *reinterpret_cast<const v8us*>(Bsrc + off);
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (ncol0 + cc + e < g.N) val[e] = Bsrc[off + e];
            }
          }
          *reinterpret_cast<v8us*>(Bl + r * 256u + cc) = val;
        }
      }
      __syncthreads();
      staged0 = grp0;
      staged1 = grp1;
    }
    if (!active) return;
    const uint32_t pbase = m0 + bi * 32u;

    // rows this lane owns in the block: 8*gq + 4*h + e, gq = 0..3, e = 0..3
    float sxv[16];
    int srcv[16];
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const uint32_t p4 = pbase + 8u * gq + 4u * h;
      const float4 s4 = *reinterpret_cast<const float4*>(g.sx + p4);
      sxv[4 * gq + 0] = s4.x; sxv[4 * gq + 1] = s4.y; sxv[4 * gq + 2] = s4.z; sxv[4 * gq + 3] = s4.w;
      if (g.src_row) {
        const int4 r4 = *reinterpret_cast<const int4*>(g.src_row + p4);
        srcv[4 * gq + 0] = r4.x; srcv[4 * gq + 1] = r4.y; srcv[4 * gq + 2] = r4.z; srcv[4 * gq + 3] = r4.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) srcv[4 * gq + e] = (int)(p4 + e);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (srcv[4 * gq + e] >= (int)g.M) srcv[4 * gq + e] = -1;
    }

    const float sgrp = has_lora ? g.lora_scaling[grp] : 0.0f;
#pragma unroll
    for (int jp = 0; jp < 2; ++jp) {
      const uint32_t ne = n0 + 64u * jp + 2u * c;  // original even column; the odd one is ne + 1
      v16f low[2];
      if (has_lora) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) low[j][e] = 0.0f;
        const uint32_t prow = pbase + c;  // A-operand row of this lane
        const int nkk = (int)(g.r_pad / 16u);
        for (int kk = 0; kk < nkk; ++kk) {
          float zf[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) zf[e] = 0.0f;
          for (uint32_t ks = 0; ks < g.ksplit; ++ks) {
            const float* zp = g.z_part + ((size_t)ks * g.slots + prow) * g.r_pad + 16u * kk + 8u * h;
            const float4 a0 = *reinterpret_cast<const float4*>(zp);
            const float4 a1 = *reinterpret_cast<const float4*>(zp + 4);
            zf[0] += a0.x; zf[1] += a0.y; zf[2] += a0.z; zf[3] += a0.w;
            zf[4] += a1.x; zf[5] += a1.y; zf[6] += a1.z; zf[7] += a1.w;
          }
          v8us zt[3];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const uint32_t b0 = f32_to_bf16_bits(zf[e]);
            const float r1 = zf[e] - bf16_bits_to_f32(b0);
            const uint32_t b1 = f32_to_bf16_bits(r1);
            const float r2 = r1 - bf16_bits_to_f32(b1);
            const uint32_t b2 = f32_to_bf16_bits(r2);
            zt[0][e] = (unsigned short)b0; zt[1][e] = (unsigned short)b1; zt[2][e] = (unsigned short)b2;
          }
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            v8us bfr;
            const uint32_t col = wn * 128u + 64u * jp + 2u * c + j;
#pragma unroll
            for (int e = 0; e < 8; ++e) bfr[e] = Bl[(16u * kk + 8u * h + e) * 256u + col];
            const v8bf bb = __builtin_bit_cast(v8bf, bfr);
            if (g.nsplit_terms >= 3)
              low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, zt[2]), bb, low[j], 0, 0, 0);
            low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, zt[1]), bb, low[j], 0, 0, 0);
            low[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, zt[0]), bb, low[j], 0, 0, 0);
          }
        }
      }
      float sw0 = 0.0f, sw1 = 0.0f;
      if (EPI != kEpiAcc) {
        if (ne < g.N) sw0 = swg[ne];
        if (ne + 1u < g.N) sw1 = swg[ne + 1u];
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int src = srcv[v];
        if (src < 0) continue;
        const int a0 = acc[bi][2 * jp][v], a1 = acc[bi][2 * jp + 1][v];
        if (EPI == kEpiAcc) {
          int32_t* o = reinterpret_cast<int32_t*>(g.out) + (size_t)src * g.N;
          if (ne < g.N) o[ne] = a0;
          if (ne + 1u < g.N) o[ne + 1u] = a1;
          continue;
        }
        float y0 = ((float)a0 * sxv[v]) * sw0;
        float y1 = ((float)a1 * sxv[v]) * sw1;
        if (has_lora) {
          const float l0 = low[0][v] * sgrp;
          const float l1 = low[1][v] * sgrp;
          y0 = y0 + l0;
          y1 = y1 + l1;
        }
        if (EPI == kEpiSwiglu) {
          const uint32_t pc = ne >> 1;
          if (pc < n_out) {
            const float gate = bf16_round_f32(y0), up = bf16_round_f32(y1);
            const float sig = 1.0f / (1.0f + __expf(-gate));
            const float prod = (gate * sig) * up;
            reinterpret_cast<uint16_t*>(g.out)[(size_t)src * n_out + pc] = (uint16_t)f32_to_bf16_bits(prod);
          }
        } else {
          uint16_t* o = reinterpret_cast<uint16_t*>(g.out) + (size_t)src * g.N;
          if (ne + 1u < g.N && (g.N & 1u) == 0) {
            if (g.residual) {
              const uint32_t rr = *reinterpret_cast<const uint32_t*>(g.residual + (size_t)src * g.N + ne);
              y0 = y0 + bf16_bits_to_f32(rr & 0xffffu);
              y1 = y1 + __uint_as_float(rr & 0xffff0000u);
            }
            *reinterpret_cast<uint32_t*>(o + ne) = f32_to_bf16_bits(y0) | (f32_to_bf16_bits(y1) << 16);
          } else {
            if (ne < g.N) {
              if (g.residual) y0 = y0 + bf16_bits_to_f32(g.residual[(size_t)src * g.N + ne]);
              o[ne] = (uint16_t)f32_to_bf16_bits(y0);
            }
            if (ne + 1u < g.N) {
              if (g.residual) y1 = y1 + bf16_bits_to_f32(g.residual[(size_t)src * g.N + ne + 1u]);
              o[ne + 1u] = (uint16_t)f32_to_bf16_bits(y1);
            }
          }
        }
      }
    }
  };
  epilogue_block(std::integral_constant<int, 0>{});
  epilogue_block(std::integral_constant<int, 1>{});
  epilogue_block(std::integral_constant<int, 2>{});
  epilogue_block(std::integral_constant<int, 3>{});
}

}  // namespace w8a8
