// Pull-backs of the two memory-bound stages around the gate/up projection of the fused
// RMSNorm -> gate/up + LoRA -> SwiGLU call
// (skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:541-574); the projection's own
// pull-back between them is the ordinary linear backward.
//
//   swiglu_bwd_kernel    (fused [M, N] bf16, d_product [M, N/2] bf16) -> d_fused [M, N] bf16
//   rms_norm_bwd_kernel  (x [M, K] bf16, gamma [K] f32, d_normalized [M, K] bf16) -> d_x [M, K] bf16
//
// Both read every operand once from HBM and write the result once.
#pragma once
#include "w8a8_device.h"

namespace w8a8 {

struct SwigluBwdArgs {
  const uint16_t* fused;   // bf16 [M, N], columns (gate_0, up_0, gate_1, up_1, ...)
  const uint16_t* dprod;   // bf16 [M, N / 2]
  uint16_t* dfused;        // bf16 [M, N]; may be the same buffer as fused
  uint64_t n_chunks;       // M * N / 8: eight projection columns = four (gate, up) pairs a chunk
};

// One (gate, up) pair, all float32, operation order of
// bf16_rms_gate_up_lora_swiglu_contiguous.py:544-552; returns d_gate | d_up << 16 as bf16 bits.
__device__ inline uint32_t swiglu_pair_pullback(float g, float u, float c) {
  const float sig = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
  const float silu = g * sig;
  const float d_up = c * silu;
  const float wc = c * u;
  const float sprime = sig * (1.0f - sig);
  const float d_gate = (wc * sig) + ((g * wc) * sprime);
  return pack_bf16x2(d_gate, d_up);
}

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(SwigluBwdArgs a) {
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < a.n_chunks; i += stride) {
    const uint4 f = *reinterpret_cast<const uint4*>(a.fused + 8u * i);
    const uint2 c = *reinterpret_cast<const uint2*>(a.dprod + 4u * i);
    uint4 o;
    o.x = swiglu_pair_pullback(__uint_as_float(f.x << 16), __uint_as_float(f.x & 0xffff0000u),
                               __uint_as_float(c.x << 16));
    o.y = swiglu_pair_pullback(__uint_as_float(f.y << 16), __uint_as_float(f.y & 0xffff0000u),
                               __uint_as_float(c.x & 0xffff0000u));
    o.z = swiglu_pair_pullback(__uint_as_float(f.z << 16), __uint_as_float(f.z & 0xffff0000u),
                               __uint_as_float(c.y << 16));
    o.w = swiglu_pair_pullback(__uint_as_float(f.w << 16), __uint_as_float(f.w & 0xffff0000u),
                               __uint_as_float(c.y & 0xffff0000u));
    *reinterpret_cast<uint4*>(a.dfused + 8u * i) = o;
  }
}

// The SwiGLU stage on its own: product[m, j] = bf16(silu(gate) * up) of the bf16 projection, the same
// arithmetic as the GEMM epilogue (bf16_rms_gate_up_lora_swiglu_contiguous.py:535-538).  A training
// forward stores the projection for the pull-back and forms the product with this kernel.
struct SwigluFwdArgs {
  const uint16_t* fused;  // bf16 [M, N]
  uint16_t* product;      // bf16 [M, N / 2]
  uint64_t n_chunks;      // M * N / 8
};

__global__ __launch_bounds__(256) void swiglu_fwd_kernel(SwigluFwdArgs a) {
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < a.n_chunks; i += stride) {
    const uint4 f = *reinterpret_cast<const uint4*>(a.fused + 8u * i);
    const uint32_t w[4] = {f.x, f.y, f.z, f.w};
    float p[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float g = __uint_as_float(w[j] << 16), u = __uint_as_float(w[j] & 0xffff0000u);
      const float sig = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
      p[j] = (g * sig) * u;
    }
    *reinterpret_cast<uint2*>(a.product + 4u * i) = make_uint2(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]));
  }
}

struct RmsNormBwdArgs {
  const uint16_t* x;    // bf16 [M, K]
  const float* gamma;   // f32 [K]: the multiplier itself (1 + delta for the Qwen3.5 flavour)
  const uint16_t* dn;   // bf16 [M, K] cotangent of the normalized activations
  uint16_t* dx;         // bf16 [M, K]; may be the same buffer as dn
  uint32_t M, K;
  float eps;
};

// Sum over the 256 threads of a workgroup; every thread gets the total.
__device__ inline double block_sum_256(double v, double* slots /* 4 */) {
  v = wave_sum(v);
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  __syncthreads();  // a previous use of the slots is over
  if (lane == 0) slots[wave] = v;
  __syncthreads();
  return (slots[0] + slots[1]) + (slots[2] + slots[3]);
}

// One workgroup per row.  With p = dn * gamma, den = mean(x^2) + eps and inv = 1 / sqrt(den):
//   t  = (sum_k x p) * (-0.5 * (inv / den)) / K
//   dx = bf16((p * inv + x * t) + t * x)
// (bf16_rms_gate_up_lora_swiglu_contiguous.py:565-573).  The mean follows the forward's rule
// (float64 sum rounded once); the row sum of x p is accumulated in float64 as well.  The second
// pass reads the row again, from L2.
template <bool VEC>
__global__ __launch_bounds__(256) void rms_norm_bwd_kernel(RmsNormBwdArgs a) {
  __shared__ double slots[4];
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  if (row >= a.M) return;
  const uint16_t* xr = a.x + (size_t)row * a.K;
  const uint16_t* dr = a.dn + (size_t)row * a.K;
  uint16_t* outr = a.dx + (size_t)row * a.K;
  double ss = 0.0, sp = 0.0;
  if (VEC) {
    for (uint32_t i = 8u * tid; i < a.K; i += 2048u) {
      const uint4 xv = *reinterpret_cast<const uint4*>(xr + i);
      const uint4 dv = *reinterpret_cast<const uint4*>(dr + i);
      const float4 g0 = *reinterpret_cast<const float4*>(a.gamma + i);
      const float4 g1 = *reinterpret_cast<const float4*>(a.gamma + i + 4u);
      const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (e & 1) ? __uint_as_float(xw[e >> 1] & 0xffff0000u) : __uint_as_float(xw[e >> 1] << 16);
        const float d = (e & 1) ? __uint_as_float(dw[e >> 1] & 0xffff0000u) : __uint_as_float(dw[e >> 1] << 16);
        const float p = d * gv[e];
        ss += (double)x * (double)x;
        sp += (double)x * (double)p;
      }
    }
  } else {
    for (uint32_t i = tid; i < a.K; i += 256u) {
      const float x = bf16_bits_to_f32(xr[i]);
      const float p = bf16_bits_to_f32(dr[i]) * a.gamma[i];
      ss += (double)x * (double)x;
      sp += (double)x * (double)p;
    }
  }
  ss = block_sum_256(ss, slots);
  sp = block_sum_256(sp, slots);
  const float mean = (float)(ss / (double)a.K);
  const float den = mean + a.eps;
  const float inv = 1.0f / sqrtf(den);
  const float ic = (float)sp;
  const float dc = ic * (-0.5f * (inv / den));
  const float t = dc / (float)a.K;
  if (VEC) {
    for (uint32_t i = 8u * tid; i < a.K; i += 2048u) {
      const uint4 xv = *reinterpret_cast<const uint4*>(xr + i);
      const uint4 dv = *reinterpret_cast<const uint4*>(dr + i);
      const float4 g0 = *reinterpret_cast<const float4*>(a.gamma + i);
      const float4 g1 = *reinterpret_cast<const float4*>(a.gamma + i + 4u);
      const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (e & 1) ? __uint_as_float(xw[e >> 1] & 0xffff0000u) : __uint_as_float(xw[e >> 1] << 16);
        const float d = (e & 1) ? __uint_as_float(dw[e >> 1] & 0xffff0000u) : __uint_as_float(dw[e >> 1] << 16);
        const float p = d * gv[e];
        o[e] = ((p * inv) + (x * t)) + (t * x);
      }
      *reinterpret_cast<uint4*>(outr + i) = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]),
                                                       pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
    }
  } else {
    for (uint32_t i = tid; i < a.K; i += 256u) {
      const float x = bf16_bits_to_f32(xr[i]);
      const float p = bf16_bits_to_f32(dr[i]) * a.gamma[i];
      outr[i] = (uint16_t)f32_to_bf16_bits(((p * inv) + (x * t)) + (t * x));
    }
  }
}

// ---------------------------------------------------------------------------------------
// The RMSNorm pull-back in the form of the Qwen3.5 attention input stage
// (_delta_rms_norm_vjp, skyrl/tx/kernels/qwen3_5_qkv_lora.py:97-116), float32:
//   n = x inv,  p = dn gamma,  mu = mean(p n),  dx = bf16(inv (p - n mu)),  dgamma = sum_rows dn n
// One workgroup per row, three passes over the row (the later ones from L2).  When inv_out is set
// the row's inv is stored for the weight-cotangent kernel below.
struct DeltaRmsBwdArgs {
  const uint16_t* x;    // bf16 [M, K]
  const float* gamma;   // f32 [K]: the multiplier 1 + weight
  const uint16_t* dn;   // bf16 [M, K]
  uint16_t* dx;         // bf16 [M, K]; may be the same buffer as dn
  float* inv_out;       // f32 [M] or null
  uint32_t M, K;
  float eps;
};

template <bool VEC>
__global__ __launch_bounds__(256) void delta_rms_norm_bwd_kernel(DeltaRmsBwdArgs a) {
  __shared__ double slots[4];
  const uint32_t row = blockIdx.x, tid = threadIdx.x;
  if (row >= a.M) return;
  const uint16_t* xr = a.x + (size_t)row * a.K;
  const uint16_t* dr = a.dn + (size_t)row * a.K;
  uint16_t* outr = a.dx + (size_t)row * a.K;
  constexpr uint32_t W = VEC ? 8u : 1u;
  double ss = 0.0;
  for (uint32_t i = W * tid; i < a.K; i += W * 256u) {
    if (VEC) {
      const uint4 xv = *reinterpret_cast<const uint4*>(xr + i);
      const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (e & 1) ? __uint_as_float(xw[e >> 1] & 0xffff0000u) : __uint_as_float(xw[e >> 1] << 16);
        ss += (double)x * (double)x;
      }
    } else {
      const float x = bf16_bits_to_f32(xr[i]);
      ss += (double)x * (double)x;
    }
  }
  ss = block_sum_256(ss, slots);
  const float mean = (float)(ss / (double)a.K);
  const float inv = 1.0f / sqrtf(mean + a.eps);
  if (a.inv_out && tid == 0) a.inv_out[row] = inv;
  double sp = 0.0;
  for (uint32_t i = W * tid; i < a.K; i += W * 256u) {
    if (VEC) {
      const uint4 xv = *reinterpret_cast<const uint4*>(xr + i);
      const uint4 dv = *reinterpret_cast<const uint4*>(dr + i);
      const float4 g0 = *reinterpret_cast<const float4*>(a.gamma + i);
      const float4 g1 = *reinterpret_cast<const float4*>(a.gamma + i + 4u);
      const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (e & 1) ? __uint_as_float(xw[e >> 1] & 0xffff0000u) : __uint_as_float(xw[e >> 1] << 16);
        const float d = (e & 1) ? __uint_as_float(dw[e >> 1] & 0xffff0000u) : __uint_as_float(dw[e >> 1] << 16);
        sp += (double)((d * gv[e]) * (x * inv));
      }
    } else {
      const float x = bf16_bits_to_f32(xr[i]);
      sp += (double)((bf16_bits_to_f32(dr[i]) * a.gamma[i]) * (x * inv));
    }
  }
  sp = block_sum_256(sp, slots);
  const float mu = (float)(sp / (double)a.K);
  for (uint32_t i = W * tid; i < a.K; i += W * 256u) {
    if (VEC) {
      const uint4 xv = *reinterpret_cast<const uint4*>(xr + i);
      const uint4 dv = *reinterpret_cast<const uint4*>(dr + i);
      const float4 g0 = *reinterpret_cast<const float4*>(a.gamma + i);
      const float4 g1 = *reinterpret_cast<const float4*>(a.gamma + i + 4u);
      const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, dw[4] = {dv.x, dv.y, dv.z, dv.w};
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (e & 1) ? __uint_as_float(xw[e >> 1] & 0xffff0000u) : __uint_as_float(xw[e >> 1] << 16);
        const float d = (e & 1) ? __uint_as_float(dw[e >> 1] & 0xffff0000u) : __uint_as_float(dw[e >> 1] << 16);
        o[e] = inv * ((d * gv[e]) - (x * inv) * mu);
      }
      *reinterpret_cast<uint4*>(outr + i) = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]),
                                                       pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
    } else {
      const float x = bf16_bits_to_f32(xr[i]);
      const float p = bf16_bits_to_f32(dr[i]) * a.gamma[i];
      outr[i] = (uint16_t)f32_to_bf16_bits(inv * (p - (x * inv) * mu));
    }
  }
}

// partial[slice][c] = sum over the rows r = slice, slice + n_slices, ... of dn[r, c] * (x[r, c] * inv[r]);
// one thread per column, gridDim = (ceil(K / 256), n_slices).  dn is the cotangent the pull-back
// above received: this kernel runs before a pull-back that overwrites it.
struct RmsDgammaArgs {
  const uint16_t* x;    // bf16 [M, K]
  const uint16_t* dn;   // bf16 [M, K]
  const float* inv;     // f32 [M]
  float* partial;       // f32 [n_slices][K]
  uint32_t M, K;
};

__global__ __launch_bounds__(256) void rms_dgamma_partial_kernel(RmsDgammaArgs a) {
  const uint32_t c = blockIdx.x * 256u + threadIdx.x;
  if (c >= a.K) return;
  float s = 0.0f;
  for (uint32_t r = blockIdx.y; r < a.M; r += gridDim.y)
    s += bf16_bits_to_f32(a.dn[(size_t)r * a.K + c]) * (bf16_bits_to_f32(a.x[(size_t)r * a.K + c]) * a.inv[r]);
  a.partial[(size_t)blockIdx.y * a.K + c] = s;
}

}  // namespace w8a8
