// Token routing around the grouped expert GEMMs (skyrl/tx/models/qwen3.py:172-210,
// skyrl/tx/layers/util.py:66-87): softmax -> top-k -> renormalise, the stable sort of
// (token, choice) pairs by expert with the gather of their rows, and the weighted sum that brings
// the expert outputs back to token order.  Index work is exact; everything is memory-bound.
//
//   moe_route_kernel           one wave per token: probabilities, top-k (ties: lower expert), weights
//   moe_route_bwd_kernel       one wave per token: the weights' cotangent back to the logits
//   moe_hist_kernel            per 1024-pair chunk: pairs per group
//   moe_scan_kernel            one workgroup: group sizes, group starts, per-chunk offsets
//   moe_scatter_kernel         per chunk: stable position of every pair, the index arrays
//   moe_gather_kernel          a wave per sorted row: the token rows copied to their positions
//   moe_spread_kernel          the same copy, a wave per token, when a token goes to several groups
//   moe_combine_kernel         one workgroup per token: sum_j expert_out[unsort[t k + j]] * w[t, j]
//   moe_combine_bwd_kernel     a wave per sorted row: the cotangents of expert_out and of w
#pragma once
#include "w8a8_device.h"

namespace w8a8 {

constexpr uint32_t kMoeMaxExperts = 1024;  // also the most groups a dispatch sorts into
constexpr uint32_t kMoeMaxTopK = 64;
constexpr uint32_t kMoeChunk = 1024;       // pairs per workgroup in the sort

// ---------------------------------------------------------------------------------------
struct MoeRouteArgs {
  const float* logits;  // f32 [T, E]
  float* weights;       // f32 [T, top_k]
  int32_t* selected;    // int32 [T, top_k]
  uint32_t T, E, top_k, norm;
};

// probabilities = exp(l - max) / sum (float32, qwen3.py:175); top_k picks the largest, the lower
// expert index on ties (lax.top_k), in descending order; weights /= their sum in selection order
// (qwen3.py:177-178).
template <uint32_t NV>  // values per lane: n_experts <= 64 * NV
__global__ __launch_bounds__(256) void moe_route_kernel(MoeRouteArgs a) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t t = blockIdx.x * 4u + wave;
  if (t >= a.T) return;
  const float* row = a.logits + (size_t)t * a.E;
  float v[NV];
  float mx = -INFINITY;
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    v[j] = e < a.E ? row[e] : -INFINITY;
    mx = fmaxf(mx, v[j]);
  }
  mx = wave_max(mx);
  float sum = 0.0f;
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    v[j] = e < a.E ? expf(v[j] - mx) : 0.0f;
    sum += v[j];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    v[j] = e < a.E ? v[j] / sum : -1.0f;  // -1: never selected
  }
  float my_w = 0.0f;
  int my_i = 0;
  for (uint32_t it = 0; it < a.top_k; ++it) {
    float best = -2.0f;
    int bi = 0x7fffffff;
#pragma unroll
    for (uint32_t j = 0; j < NV; ++j)
      if (v[j] > best) { best = v[j]; bi = (int)(j * 64u + lane); }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off);
      const int oi = __shfl_xor(bi, off);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (lane == ((uint32_t)bi & 63u)) {
#pragma unroll
      for (uint32_t j = 0; j < NV; ++j)
        if (j == ((uint32_t)bi >> 6)) v[j] = -1.0f;
    }
    if (lane == it) { my_w = best; my_i = bi; }
  }
  if (a.norm) {
    float s = 0.0f;
    for (uint32_t j = 0; j < a.top_k; ++j) {
      const float wj = __shfl(my_w, (int)j);
      s = j == 0 ? wj : s + wj;
    }
    my_w = my_w / s;
  }
  if (lane < a.top_k) {
    a.weights[(size_t)t * a.top_k + lane] = my_w;
    a.selected[(size_t)t * a.top_k + lane] = my_i;
  }
}

// Pull-back of the routing weights to the router logits with the selection held fixed (lax.top_k
// has no derivative in its indices): p = softmax(l); ps = p[selected]; w = ps / sum(ps) when
// normalised;  d_ps = (d_w - sum(d_w w)) / sum(ps)  (or d_w);  d_l = p (d_p - sum(p d_p)) with d_p
// zero outside the selection (qwen3.py:175-178).  One wave per token, float32.
struct MoeRouteBwdArgs {
  const float* logits;     // f32 [T, E]
  const int32_t* selected; // int32 [T, top_k]
  const float* d_weights;  // f32 [T, top_k]
  float* d_logits;         // f32 [T, E]
  uint32_t T, E, top_k, norm;
};

template <uint32_t NV>
__global__ __launch_bounds__(256) void moe_route_bwd_kernel(MoeRouteBwdArgs a) {
  __shared__ float tab[4][kMoeMaxExperts];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t t = blockIdx.x * 4u + wave;
  if (t >= a.T) return;
  const float* row = a.logits + (size_t)t * a.E;
  float v[NV];
  float mx = -INFINITY;
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    v[j] = e < a.E ? row[e] : -INFINITY;
    mx = fmaxf(mx, v[j]);
  }
  mx = wave_max(mx);
  float sum = 0.0f;
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    v[j] = e < a.E ? expf(v[j] - mx) : 0.0f;
    sum += v[j];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    v[j] = v[j] / sum;
    if (e < a.E) tab[wave][e] = v[j];
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave reads what its own lanes wrote
  __builtin_amdgcn_wave_barrier();
  // lane j < top_k owns choice j
  const bool own = lane < a.top_k;
  const int sel = own ? a.selected[(size_t)t * a.top_k + lane] : 0;
  const uint32_t se = sel < 0 ? 0u : ((uint32_t)sel >= a.E ? a.E - 1u : (uint32_t)sel);
  const float dw = own ? a.d_weights[(size_t)t * a.top_k + lane] : 0.0f;
  const float ps = own ? tab[wave][se] : 0.0f;
  float dps = dw;
  if (a.norm) {
    float tot = ps, dot = 0.0f;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) tot += __shfl_xor(tot, off);
    dot = dw * (ps / tot);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
    dps = (dw - dot) / tot;
  }
  float s = own ? ps * dps : 0.0f;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
  __builtin_amdgcn_wave_barrier();  // every lane has read its probability
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    if (e < a.E) tab[wave][e] = 0.0f;
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_wave_barrier();
  if (own) tab[wave][se] = dps;  // the selection holds distinct experts
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (uint32_t j = 0; j < NV; ++j) {
    const uint32_t e = j * 64u + lane;
    if (e < a.E) a.d_logits[(size_t)t * a.E + e] = v[j] * (tab[wave][e] - s);
  }
}

// ---------------------------------------------------------------------------------------
struct MoeSortArgs {
  const int32_t* indices;   // int32 [P] group of every pair (clamped into range)
  const uint16_t* tokens;   // bf16 [P / repeat, width] or null (indices only)
  const int32_t* adapters;  // int32 [P / repeat] or null
  uint16_t* sorted_tokens;  // bf16 [P, width]
  int32_t* group_sizes;     // int32 [G]
  int32_t* sort_indices;    // int32 [P]: pair at every sorted position
  int32_t* unsort_indices;  // int32 [P]: sorted position of every pair
  int32_t* sorted_adapters; // int32 [P] or null
  int32_t* chunk_cnt;       // workspace int32 [n_chunks][G]: counts, then offsets inside the group
  int32_t* group_start;     // workspace int32 [G]
  uint32_t P, G, repeat, width, n_chunks;
};

__device__ inline uint32_t moe_group_of(const MoeSortArgs& a, uint32_t p) {
  const int g = a.indices[p];
  return g < 0 ? 0u : (g >= (int)a.G ? a.G - 1u : (uint32_t)g);
}

__global__ __launch_bounds__(1024) void moe_hist_kernel(MoeSortArgs a) {
  __shared__ int cnt[kMoeMaxExperts];
  const uint32_t tid = threadIdx.x, chunk = blockIdx.x;
  if (tid < a.G) cnt[tid] = 0;
  __syncthreads();
  const uint32_t p = chunk * kMoeChunk + tid;
  if (p < a.P) atomicAdd(&cnt[moe_group_of(a, p)], 1);
  __syncthreads();
  if (tid < a.G) a.chunk_cnt[(size_t)chunk * a.G + tid] = cnt[tid];
}

__global__ __launch_bounds__(1024) void moe_scan_kernel(MoeSortArgs a) {
  __shared__ int scan[kMoeMaxExperts];
  const uint32_t g = threadIdx.x;
  int run = 0;
  if (g < a.G) {
#pragma unroll 8
    for (uint32_t c = 0; c < a.n_chunks; ++c) {
      const int t = a.chunk_cnt[(size_t)c * a.G + g];
      a.chunk_cnt[(size_t)c * a.G + g] = run;
      run += t;
    }
    a.group_sizes[g] = run;
  }
  scan[g] = run;
  __syncthreads();
  for (uint32_t off = 1; off < kMoeMaxExperts; off <<= 1) {
    const int add = g >= off ? scan[g - off] : 0;
    __syncthreads();
    scan[g] += add;
    __syncthreads();
  }
  if (g < a.G) a.group_start[g] = scan[g] - run;  // exclusive
}

// Position of pair p = start of its group + pairs of the group in earlier chunks + pairs of the
// group earlier in this chunk (earlier waves, then earlier lanes of its wave): a stable sort.
__global__ __launch_bounds__(1024) void moe_scatter_kernel(MoeSortArgs a) {
  __shared__ uint16_t wave_cnt[16][kMoeMaxExperts];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, chunk = blockIdx.x;
  for (uint32_t i = tid; i < 16u * a.G; i += 1024u) wave_cnt[i / a.G][i % a.G] = 0;
  __syncthreads();
  const uint32_t p = chunk * kMoeChunk + tid;
  const bool valid = p < a.P;
  const uint32_t g = valid ? moe_group_of(a, p) : 0u;
  // the lanes of this wave that hold the same group: one ballot per bit of the group index
  // (at most ten), instead of one round per distinct group
  unsigned long long same = __builtin_amdgcn_ballot_w64(valid);
  for (uint32_t bit = 0; (1u << bit) < a.G; ++bit) {  // wave-uniform trip count
    const bool one = (g >> bit) & 1u;
    const unsigned long long ones = __builtin_amdgcn_ballot_w64(one);
    same &= one ? ones : ~ones;
  }
  const uint32_t rank = (uint32_t)__builtin_popcountll(same & ((1ull << lane) - 1ull));
  if (valid && rank == 0) wave_cnt[wave][g] = (uint16_t)__builtin_popcountll(same);
  __syncthreads();
  if (valid) {
    uint32_t before = 0;
    for (uint32_t w = 0; w < wave; ++w) before += wave_cnt[w][g];
    const int pos = a.group_start[g] + a.chunk_cnt[(size_t)chunk * a.G + g] + (int)before + (int)rank;
    a.sort_indices[pos] = (int)p;
    a.unsort_indices[p] = pos;
    if (a.sorted_adapters) a.sorted_adapters[pos] = a.adapters[p / a.repeat];
  }
}

// sorted_tokens[pos] = tokens[sort_indices[pos] / repeat]: a wave per row, two rows a wave.
__global__ __launch_bounds__(256) void moe_gather_kernel(MoeSortArgs a) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
#pragma unroll
  for (uint32_t u = 0; u < 2; ++u) {
    const uint32_t pos = blockIdx.x * 8u + wave * 2u + u;
    if (pos >= a.P) return;
    const uint16_t* src = a.tokens + (size_t)((uint32_t)a.sort_indices[pos] / a.repeat) * a.width;
    uint16_t* out = a.sorted_tokens + (size_t)pos * a.width;
    for (uint32_t c = lane * 8u; c < a.width; c += 512u)
      *reinterpret_cast<uint4*>(out + c) = *reinterpret_cast<const uint4*>(src + c);
  }
}

// The same rows written from the token's side when every token goes to several groups
// (repeat > 1): sorted_tokens[unsort_indices[t * repeat + j]] = tokens[t].  A wave per token
// reads the row once and stores it `repeat` times; the gather form reads it once per pair,
// and those reads miss the caches because the copies of a token lie far apart in the sorted order.
__global__ __launch_bounds__(256) void moe_spread_kernel(MoeSortArgs a) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t t = blockIdx.x * 4u + wave;
  if (t >= a.P / a.repeat) return;
  const uint16_t* src = a.tokens + (size_t)t * a.width;
  const int32_t* dst = a.unsort_indices + (size_t)t * a.repeat;
  for (uint32_t c0 = lane * 8u; c0 < a.width; c0 += 2048u) {  // four 16-byte pieces per lane and round
    uint4 v[4];
#pragma unroll
    for (uint32_t u = 0; u < 4; ++u)
      if (c0 + u * 512u < a.width) v[u] = *reinterpret_cast<const uint4*>(src + c0 + u * 512u);
    for (uint32_t j = 0; j < a.repeat; ++j) {
      uint16_t* out = a.sorted_tokens + (size_t)(uint32_t)dst[j] * a.width;
#pragma unroll
      for (uint32_t u = 0; u < 4; ++u)
        if (c0 + u * 512u < a.width) *reinterpret_cast<uint4*>(out + c0 + u * 512u) = v[u];
    }
  }
}

// ---------------------------------------------------------------------------------------
struct MoeCombineArgs {
  const uint16_t* expert_out;  // bf16 [P, width] in sorted order
  const int32_t* unsort;       // int32 [P]
  const float* weights;        // f32 [T, top_k]
  uint16_t* out;               // bf16 [T, width]
  uint32_t T, top_k, width;
};

// out[t] = bf16(sum_j f32(expert_out[unsort[t k + j]]) * w[t, j]), products and the sum in float32 in
// choice order, one cast (qwen3.py:205-207 with the float32 policy of this path).
__global__ __launch_bounds__(256) void moe_combine_kernel(MoeCombineArgs a) {
  __shared__ int rows[kMoeMaxTopK];
  __shared__ float w[kMoeMaxTopK];
  const uint32_t t = blockIdx.x, tid = threadIdx.x;
  if (t >= a.T) return;
  if (tid < a.top_k) {
    rows[tid] = a.unsort[(size_t)t * a.top_k + tid];
    w[tid] = a.weights[(size_t)t * a.top_k + tid];
  }
  __syncthreads();
  for (uint32_t c = tid * 8u; c < a.width; c += 2048u) {
    float acc[8];
    for (uint32_t j = 0; j < a.top_k; ++j) {
      const uint4 raw = *reinterpret_cast<const uint4*>(a.expert_out + (size_t)rows[j] * a.width + c);
      const uint32_t rw[4] = {raw.x, raw.y, raw.z, raw.w};
      const float wj = w[j];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = (e & 1) ? __uint_as_float(rw[e >> 1] & 0xffff0000u) : __uint_as_float(rw[e >> 1] << 16);
        const float prod = x * wj;
        acc[e] = j == 0 ? prod : acc[e] + prod;
      }
    }
    *reinterpret_cast<uint4*>(a.out + (size_t)t * a.width + c) =
        make_uint4(pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]), pack_bf16x2(acc[4], acc[5]),
                   pack_bf16x2(acc[6], acc[7]));
  }
}

// ---------------------------------------------------------------------------------------
// Pull-back of the combine: for the sorted row at position pos, with pair = sort[pos] (token
// pair / top_k, weight w[pair]):
//   d_expert_out[pos] = bf16(f32(d_out[token]) * w[pair])
//   d_weights[pair]   = sum_c f32(expert_out[pos, c]) * f32(d_out[token, c])      (float32)
// the derivative of out[t] = sum_j expert_out[unsort[t k + j]] * w[t, j] (qwen3.py:205-207).  A wave
// per sorted row; the dot product is summed per lane, then across the wave.
struct MoeCombineBwdArgs {
  const uint16_t* d_out;       // bf16 [T, width]
  const uint16_t* expert_out;  // bf16 [P, width] in sorted order, or null (no weight cotangent)
  const int32_t* sort;         // int32 [P]
  const float* weights;        // f32 [T, top_k]
  uint16_t* d_expert_out;      // bf16 [P, width]
  float* d_weights;            // f32 [T, top_k] or null
  uint32_t P, top_k, width;
};

__global__ __launch_bounds__(256) void moe_combine_bwd_kernel(MoeCombineBwdArgs a) {
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
#pragma unroll
  for (uint32_t u = 0; u < 2; ++u) {
    const uint32_t pos = blockIdx.x * 8u + wave * 2u + u;
    if (pos >= a.P) return;
    const uint32_t pair = (uint32_t)a.sort[pos];
    const float w = a.weights[pair];
    const uint16_t* src = a.d_out + (size_t)(pair / a.top_k) * a.width;
    const uint16_t* eo = a.expert_out ? a.expert_out + (size_t)pos * a.width : nullptr;
    uint16_t* out = a.d_expert_out + (size_t)pos * a.width;
    float dot = 0.0f;
    for (uint32_t c = lane * 8u; c < a.width; c += 512u) {
      const uint4 raw = *reinterpret_cast<const uint4*>(src + c);
      const uint32_t rw[4] = {raw.x, raw.y, raw.z, raw.w};
      uint32_t ew[4] = {0, 0, 0, 0};
      if (eo) {
        const uint4 er = *reinterpret_cast<const uint4*>(eo + c);
        ew[0] = er.x; ew[1] = er.y; ew[2] = er.z; ew[3] = er.w;
      }
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = (e & 1) ? __uint_as_float(rw[e >> 1] & 0xffff0000u) : __uint_as_float(rw[e >> 1] << 16);
        const float x = (e & 1) ? __uint_as_float(ew[e >> 1] & 0xffff0000u) : __uint_as_float(ew[e >> 1] << 16);
        o[e] = d * w;
        dot += x * d;
      }
      *reinterpret_cast<uint4*>(out + c) =
          make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
    }
    if (a.d_weights) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
      if (lane == 0) a.d_weights[pair] = dot;
    }
  }
}

}  // namespace w8a8
