// Qwen3.5 attention input stage behind the fused QKV projection
// (skyrl/tx/kernels/qwen3_5_qkv_lora.py:216-286): split the interleaved projection, RMSNorm with
// (1 + weight) over every Q and K head, partial RoPE on Q and K, V and the Q gates copied out.
// The projection itself (RMSNorm prologue, W8A8 GEMM, LoRA) is the ordinary forward call; this
// kernel reads its bf16 output once and writes q, k, v, gate once (memory-bound).
//
// Layout of a fused row: per kv head one group [q_0 g_0 ... q_{qpk-1} g_{qpk-1} k v], every chunk
// head_dim wide (qwen3_5_qkv_lora.py:40-46).  One workgroup per row; a wave takes a (q, gate) or a
// (k, v) pair at a time.
#pragma once
#include "w8a8_device.h"

namespace w8a8 {

constexpr uint32_t kQkvMaxHeadDim = 512;

struct QkvPostArgs {
  const uint16_t* fused;   // bf16 [M, width]
  const float* q_w;        // f32 [D] delta weights of the Q norm
  const float* k_w;        // f32 [D]
  const int32_t* pos;      // int32 [M]
  uint16_t* q;             // bf16 [M, Hq, D]
  uint16_t* k;             // bf16 [M, Hkv, D]
  uint16_t* v;             // bf16 [M, Hkv, D]
  uint16_t* gate;          // bf16 [M, Hq * D]
  uint32_t M, Hq, Hkv, D, rot, width;
  float theta, eps;
};

__global__ __launch_bounds__(256) void qkv_post_kernel(QkvPostArgs a) {
  __shared__ float sn[kQkvMaxHeadDim / 2], cs[kQkvMaxHeadDim / 2];
  __shared__ float buf[4][kQkvMaxHeadDim];
  const uint32_t row = blockIdx.x, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  if (row >= a.M) return;
  const uint32_t half = a.rot / 2u;
  // angle[i] = position / theta^(2 i / rot), all float32 (qwen3_5_qkv_lora.py:119-127)
  const float position = (float)a.pos[row];
  for (uint32_t i = tid; i < half; i += 256u) {
    const float fraction = (2.0f * (float)i) / (float)a.rot;
    const float angle = position / powf(a.theta, fraction);
    sn[i] = sinf(angle);
    cs[i] = cosf(angle);
  }
  __syncthreads();
  const uint32_t qpk = a.Hq / a.Hkv;
  const uint32_t group_width = (qpk * 2u + 2u) * a.D;
  const uint16_t* frow = a.fused + (size_t)row * a.width;
  const uint32_t units = a.Hq + a.Hkv;
  // four consecutive elements per lane (8-byte accesses) where the geometry allows it
  const bool vec4 = (a.D & 3u) == 0 && (half & 3u) == 0 && (a.width & 3u) == 0;
  for (uint32_t u = wave; u < units; u += 4u) {  // wave-uniform
    const bool is_q = u < a.Hq;
    const uint32_t g = is_q ? u / qpk : u - a.Hq;
    const uint32_t off = g * group_width + (is_q ? (u % qpk) * 2u * a.D : qpk * 2u * a.D);
    const float* w = is_q ? a.q_w : a.k_w;
    uint16_t* normed = is_q ? a.q + ((size_t)row * a.Hq + u) * a.D : a.k + ((size_t)row * a.Hkv + g) * a.D;
    uint16_t* copied = is_q ? a.gate + ((size_t)row * a.Hq + u) * a.D : a.v + ((size_t)row * a.Hkv + g) * a.D;
    if (vec4) {
      // the second chunk of the pair (gate or v) passes through
      for (uint32_t i = 4u * lane; i < a.D; i += 256u)
        *reinterpret_cast<uint2*>(copied + i) = *reinterpret_cast<const uint2*>(frow + off + a.D + i);
      // RMSNorm over the head: mean = float(sum_f64(x^2) / D), inv = 1 / sqrt(mean + eps) (IEEE),
      // n = bf16((x * inv) * (1 + w)); D <= 512: at most two pieces per lane, kept in registers
      uint2 raw[2] = {make_uint2(0, 0), make_uint2(0, 0)};
      double ss = 0.0;
#pragma unroll
      for (uint32_t j = 0; j < 2; ++j) {
        const uint32_t i = 4u * lane + 256u * j;
        if (i < a.D) {
          raw[j] = *reinterpret_cast<const uint2*>(frow + off + i);
          const float x0 = __uint_as_float(raw[j].x << 16), x1 = __uint_as_float(raw[j].x & 0xffff0000u);
          const float x2 = __uint_as_float(raw[j].y << 16), x3 = __uint_as_float(raw[j].y & 0xffff0000u);
          ss += (double)x0 * (double)x0 + (double)x1 * (double)x1 + (double)x2 * (double)x2 + (double)x3 * (double)x3;
        }
      }
      ss = wave_sum(ss);
      const float mean = (float)(ss / (double)a.D);
      const float inv = 1.0f / sqrtf(mean + a.eps);
#pragma unroll
      for (uint32_t j = 0; j < 2; ++j) {
        const uint32_t i = 4u * lane + 256u * j;
        if (i < a.D) {
          const float4 w4 = *reinterpret_cast<const float4*>(w + i);
          const float x[4] = {__uint_as_float(raw[j].x << 16), __uint_as_float(raw[j].x & 0xffff0000u),
                              __uint_as_float(raw[j].y << 16), __uint_as_float(raw[j].y & 0xffff0000u)};
          const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
          float4 n4;
          float* np_ = &n4.x;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float t = x[e] * inv;
            t = t * (1.0f + wv[e]);
            np_[e] = bf16_round_f32(t);
          }
          *reinterpret_cast<float4*>(&buf[wave][i]) = n4;
        }
      }
      // the wave reads what other lanes of the same wave wrote: LDS operations of a wave complete
      // in order, the barrier-free hand-over only needs them drained
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (uint32_t j = 0; j < 2; ++j) {
        const uint32_t i = 4u * lane + 256u * j;
        if (i < a.D) {
          float4 o4 = *reinterpret_cast<const float4*>(&buf[wave][i]);
          if (i < a.rot) {
            // halves (i, i + rot / 2): [first cos - second sin, first sin + second cos], products in float32
            float* o = &o4.x;
            if (i < half) {
              const float4 s2 = *reinterpret_cast<const float4*>(&buf[wave][i + half]);
              const float* sp = &s2.x;
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = o[e] * cs[i + e] - sp[e] * sn[i + e];
            } else {
              const float4 f2 = *reinterpret_cast<const float4*>(&buf[wave][i - half]);
              const float* fp = &f2.x;
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = fp[e] * sn[i - half + e] + o[e] * cs[i - half + e];
            }
          }
          *reinterpret_cast<uint2*>(normed + i) = make_uint2(pack_bf16x2(o4.x, o4.y), pack_bf16x2(o4.z, o4.w));
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();  // buf[wave] is rewritten by the next unit
      continue;
    }
    // general geometry: one element per lane and step
    for (uint32_t i = lane; i < a.D; i += 64u) copied[i] = frow[off + a.D + i];
    double ss = 0.0;
    for (uint32_t i = lane; i < a.D; i += 64u) {
      const float x = bf16_bits_to_f32(frow[off + i]);
      ss += (double)x * (double)x;
    }
    ss = wave_sum(ss);
    const float mean = (float)(ss / (double)a.D);
    const float inv = 1.0f / sqrtf(mean + a.eps);
    for (uint32_t i = lane; i < a.D; i += 64u) {
      const float x = bf16_bits_to_f32(frow[off + i]);
      float t = x * inv;
      t = t * (1.0f + w[i]);
      buf[wave][i] = bf16_round_f32(t);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    for (uint32_t i = lane; i < a.D; i += 64u) {
      float o = buf[wave][i];
      if (i < a.rot) {
        if (i < half) o = buf[wave][i] * cs[i] - buf[wave][i + half] * sn[i];
        else o = buf[wave][i - half] * sn[i - half] + buf[wave][i] * cs[i - half];
      }
      normed[i] = (uint16_t)f32_to_bf16_bits(o);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
  }
}

// ---------------------------------------------------------------------------------------
// Pull-back of the kernel above (qwen3_5_qkv_lora.py:391-425): the transposed partial rotation on
// the Q and K cotangents, the RMSNorm pull-back of every Q and K head against the raw projection,
// and the re-interleave with the gate and V cotangents into the cotangent of the fused projection.
// Optionally the cotangents of the two head-norm weights (sums over rows and heads).
//
// Per head, float32 in the order of _apply_partial_rope_transpose (:148-164) and
// _delta_rms_norm_vjp (:97-116):
//   u  = bf16([first cos + second sin, second cos - first sin]) on the rotated part of dy
//   n  = x inv,  p = u (1 + w),  mu = mean(p n),  dx = bf16(inv (p - n mu)),  dw += u n
struct QkvPostBwdArgs {
  const uint16_t* fused;   // bf16 [M, width] raw projection
  const float* q_w;        // f32 [D]
  const float* k_w;        // f32 [D]
  const int32_t* pos;      // int32 [M]
  const uint16_t* dq;      // bf16 [M, Hq, D]
  const uint16_t* dk;      // bf16 [M, Hkv, D]
  const uint16_t* dv;      // bf16 [M, Hkv, D]
  const uint16_t* dgate;   // bf16 [M, Hq * D]
  uint16_t* dfused;        // bf16 [M, width]
  float* partial;          // f32 [gridDim.x][2][D] when the weight cotangents are wanted
  uint32_t M, Hq, Hkv, D, rot, width;
  float theta, eps;
};

// V consecutive elements per lane and piece (V = 4: 8-byte accesses; V = 1: any geometry); a head
// has at most kQkvMaxHeadDim / (64 V) pieces per lane.  Workgroups stride over the rows so that the
// weight cotangents accumulate in registers; WGRAD = false leaves them out altogether.
template <int V, bool WGRAD>
__global__ __launch_bounds__(256) void qkv_post_bwd_kernel(QkvPostBwdArgs a) {
  constexpr uint32_t NP = kQkvMaxHeadDim / (64u * V);
  __shared__ float sn[kQkvMaxHeadDim / 2], cs[kQkvMaxHeadDim / 2];
  __shared__ float buf[4][kQkvMaxHeadDim];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t half = a.rot / 2u;
  const uint32_t qpk = a.Hq / a.Hkv;
  const uint32_t group_width = (qpk * 2u + 2u) * a.D;
  const uint32_t units = a.Hq + a.Hkv;
  float wq[NP * V], wk[NP * V];
#pragma unroll
  for (uint32_t e = 0; e < NP * V; ++e) wq[e] = wk[e] = 0.0f;

  for (uint32_t row = blockIdx.x; row < a.M; row += gridDim.x) {
    __syncthreads();  // the tables of the previous row are no longer read
    const float position = (float)a.pos[row];
    for (uint32_t i = tid; i < half; i += 256u) {
      const float fraction = (2.0f * (float)i) / (float)a.rot;
      const float angle = position / powf(a.theta, fraction);
      sn[i] = sinf(angle);
      cs[i] = cosf(angle);
    }
    __syncthreads();
    const uint16_t* frow = a.fused + (size_t)row * a.width;
    uint16_t* orow = a.dfused + (size_t)row * a.width;
    for (uint32_t u = wave; u < units; u += 4u) {  // wave-uniform
      const bool is_q = u < a.Hq;
      const uint32_t g = is_q ? u / qpk : u - a.Hq;
      const uint32_t off = g * group_width + (is_q ? (u % qpk) * 2u * a.D : qpk * 2u * a.D);
      const float* w = is_q ? a.q_w : a.k_w;
      const uint16_t* dy = is_q ? a.dq + ((size_t)row * a.Hq + u) * a.D : a.dk + ((size_t)row * a.Hkv + g) * a.D;
      const uint16_t* dcopy = is_q ? a.dgate + ((size_t)row * a.Hq + u) * a.D : a.dv + ((size_t)row * a.Hkv + g) * a.D;
      float x[NP * V], d[NP * V];
      double ss = 0.0;
#pragma unroll
      for (uint32_t j = 0; j < NP; ++j) {
        const uint32_t i = V * lane + 64u * V * j;
        if (i < a.D) {
          if constexpr (V == 4) {
            *reinterpret_cast<uint2*>(orow + off + a.D + i) = *reinterpret_cast<const uint2*>(dcopy + i);
            const uint2 xr = *reinterpret_cast<const uint2*>(frow + off + i);
            const uint2 dr = *reinterpret_cast<const uint2*>(dy + i);
            x[4 * j + 0] = __uint_as_float(xr.x << 16); x[4 * j + 1] = __uint_as_float(xr.x & 0xffff0000u);
            x[4 * j + 2] = __uint_as_float(xr.y << 16); x[4 * j + 3] = __uint_as_float(xr.y & 0xffff0000u);
            d[4 * j + 0] = __uint_as_float(dr.x << 16); d[4 * j + 1] = __uint_as_float(dr.x & 0xffff0000u);
            d[4 * j + 2] = __uint_as_float(dr.y << 16); d[4 * j + 3] = __uint_as_float(dr.y & 0xffff0000u);
          } else {
            orow[off + a.D + i] = dcopy[i];
            x[j] = bf16_bits_to_f32(frow[off + i]);
            d[j] = bf16_bits_to_f32(dy[i]);
          }
#pragma unroll
          for (int e = 0; e < V; ++e) {
            ss += (double)x[V * j + e] * (double)x[V * j + e];
            buf[wave][i + e] = d[V * j + e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e) x[V * j + e] = d[V * j + e] = 0.0f;
        }
      }
      ss = wave_sum(ss);
      const float mean = (float)(ss / (double)a.D);
      const float inv = 1.0f / sqrtf(mean + a.eps);
      // the rotation pairs element i with i +- rot / 2, held by another lane of this wave
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_wave_barrier();
      float n[NP * V], p[NP * V];
      double sp = 0.0;
#pragma unroll
      for (uint32_t j = 0; j < NP; ++j) {
        const uint32_t i = V * lane + 64u * V * j;
        if (i < a.D) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            const uint32_t c = i + e;
            float uo = d[V * j + e];
            if (c < a.rot) {
              if (c < half) uo = uo * cs[c] + buf[wave][c + half] * sn[c];
              else uo = uo * cs[c - half] - buf[wave][c - half] * sn[c - half];
              uo = bf16_round_f32(uo);
            }
            d[V * j + e] = uo;
            n[V * j + e] = x[V * j + e] * inv;
            p[V * j + e] = uo * (1.0f + w[c]);
            sp += (double)(p[V * j + e] * n[V * j + e]);
          }
        }
      }
      sp = wave_sum(sp);
      const float mu = (float)(sp / (double)a.D);
#pragma unroll
      for (uint32_t j = 0; j < NP; ++j) {
        const uint32_t i = V * lane + 64u * V * j;
        if (i < a.D) {
          float o[V];
#pragma unroll
          for (int e = 0; e < V; ++e) {
            o[e] = inv * (p[V * j + e] - n[V * j + e] * mu);
            if (WGRAD) {
              const float t = d[V * j + e] * n[V * j + e];
              wq[V * j + e] += is_q ? t : 0.0f;
              wk[V * j + e] += is_q ? 0.0f : t;
            }
          }
          if constexpr (V == 4) {
            *reinterpret_cast<uint2*>(orow + off + i) = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
          } else {
            orow[off + i] = (uint16_t)f32_to_bf16_bits(o[0]);
          }
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();  // buf[wave] is rewritten by the next unit
    }
  }
  if (WGRAD) {
    // the four waves' sums, wave 0 first; buf is free once every wave is past its rows
    for (uint32_t which = 0; which < 2; ++which) {
      __syncthreads();
#pragma unroll
      for (uint32_t j = 0; j < NP; ++j) {
        const uint32_t i = V * lane + 64u * V * j;
        if (i < a.D) {
#pragma unroll
          for (int e = 0; e < V; ++e) buf[wave][i + e] = which == 0 ? wq[V * j + e] : wk[V * j + e];
        }
      }
      __syncthreads();
      for (uint32_t i = tid; i < a.D; i += 256u)
        a.partial[((size_t)blockIdx.x * 2u + which) * a.D + i] = ((buf[0][i] + buf[1][i]) + buf[2][i]) + buf[3][i];
    }
  }
}

// out[c] = sum over the n_parts rows of partial[part][col0 + c].  A workgroup takes 16 columns; its
// 16 lanes per column sum every 16th part each (lane l: parts l, l + 16, ...), then lane 0 adds the
// 16 sums in lane order: a fixed order whatever the launch.
struct ColumnSumArgs {
  const float* partial;  // f32 [n_parts][stride]
  float* out;            // f32 [cols]
  uint32_t n_parts, stride, cols, col0;
};

__global__ __launch_bounds__(256) void column_sum_kernel(ColumnSumArgs a) {
  __shared__ float red[16][17];
  const uint32_t cl = threadIdx.x & 15u, pl = threadIdx.x >> 4;
  const uint32_t c = blockIdx.x * 16u + cl;
  float s = 0.0f;
  if (c < a.cols) {
#pragma unroll 4
    for (uint32_t p = pl; p < a.n_parts; p += 16u) s += a.partial[(size_t)p * a.stride + a.col0 + c];
  }
  red[pl][cl] = s;
  __syncthreads();
  if (pl == 0 && c < a.cols) {
    float t = red[0][cl];
#pragma unroll
    for (uint32_t l = 1; l < 16; ++l) t += red[l][cl];
    a.out[c] = t;
  }
}

}  // namespace w8a8
