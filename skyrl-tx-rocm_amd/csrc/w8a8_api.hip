// C ABI of the MI355X W8A8 LoRA linear forward path: argument validation, workspace
// carving and kernel launches.  Nothing here synchronises, allocates or keeps state.
#include "../../include/mi355_w8a8.h"

#include <hip/hip_runtime.h>

#include <mutex>

#include "w8a8_device.h"
#include "w8a8_gemm.h"
#include "w8a8_gemm16.h"
#include "w8a8_calibration.h"
#include "w8a8_prologue.h"
#include "w8a8_skinny.h"
#include "w8a8_backward.h"
#include "w8a8_qkv_post.h"
#include "w8a8_fused_bwd.h"
#include "w8a8_moe.h"
#include "w8a8_gq.h"

using namespace w8a8;

// Workspace of mi355_w8a8_forward_static_ws_v1: one copy per GPU, held until the process ends.  In host
// code this name is a stand-in, not a device address: the per-device address comes from
// hipGetSymbolAddress (static_workspace() below) and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[MI355_W8A8_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up once per device), or null.
void* static_workspace() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

constexpr uint32_t kMaxK = 16384;
constexpr uint32_t kMaxRows = 1u << 20;
constexpr uint32_t kMaxN = 1u << 20;

inline uint64_t align256(uint64_t v) { return (v + 255u) & ~uint64_t(255); }

struct WsLayout {
  uint64_t xq, sx, xn, zp, at, bp, src_row, dst_pos, slot_group, blk_range, tile_ctr, skinny, total;
  uint32_t slots, nkk, K_pad, KB, n_steps, steps_per_wave;
  uint32_t rows_bound;  // the slots that can hold rows (a multiple of 32)
};

// number of 16-wide rank chunks the kernels are instantiated for (rank padded with zeros)
inline uint32_t rank_chunks(uint32_t rank) { return rank == 0 ? 0u : (rank <= 16u ? 1u : (rank <= 32u ? 2u : 4u)); }

// Between the skinny-M limit and this many rows a call without SwiGLU may run the skinny-M kernels
// on chunks of 32 rows: the weight is streamed once per chunk (the later passes from the last-level
// cache).  A chunk costs 14-29 us, growing with the weight's bytes; the tiled call (128 x 128 tiles,
// adapters on block boundaries) about 20 us + 7.5 us per 1024 of K whatever the rows.  Measured,
// chunks against tiles: 4096 x 2560 at 64 rows 43 us / 57, at 96 rows 63 / 57; 12288 x 4096 at
// 96 rows 88 / 113, at 128 rows 116 / 114; 2560 x 6144 at 33 rows 55 / 42; 1024 x 1024 at 33 rows 27 / 24.
constexpr uint32_t kSkinnyChunkedMaxRows = 128;
inline bool skinny_chunked_pays(uint32_t m, uint32_t k, uint32_t n) {
  if (m > kSkinnyChunkedMaxRows || (uint64_t)k_padded(k) * n_padded(n) > (64ull << 20)) return false;
  if (k < 4096u) return false;
  if (k >= 8192u) return m <= 96u;
  return m <= 64u && n_padded(n) <= 4096u;
}

// Grouped slots a call of m rows and n_groups adapters can need when every adapter's rows start on a
// 32-slot block boundary (sum of the groups' sizes rounded up to 32).
inline uint32_t padded_rows_bound(uint32_t m, uint32_t n_groups) {
  return round_up(m + 31u * (n_groups < m ? n_groups : m), 32u);
}
// Whether a routed call may lay its groups out that way: the quantizer sorts the rows itself, and the
// empty slots cost no time -- neither the quantizer's workgroups (16 slots each, one resident per CU) nor
// the GEMM's tiles (512 resident tiles of 128 x 128, 256 of 256 x 256) need another round on the chip
// than the packed layout does.
inline bool padded_groups_fit(uint32_t m, uint32_t n, uint32_t n_groups, bool wide_tiles = false) {
  if (n_groups < 2u || m > kInlineRouteMaxRows) return false;
  const uint32_t rows = padded_rows_bound(m, n_groups), base = round_up(m, 32u);
  auto rounds = [](uint64_t items, uint64_t resident) { return (items + resident - 1u) / resident; };
  if (rounds(rows / 16u, 256u) != rounds(base / 16u, 256u)) return false;
  const uint32_t tile_m = wide_tiles ? (uint32_t)kTileM : (uint32_t)kGemm128TileM;
  const uint64_t per_row = n_padded(n) / (wide_tiles ? (uint32_t)kG16TileN : (uint32_t)kGemmTileN);
  const uint64_t resident = wide_tiles ? 256u : 512u;
  return rounds((uint64_t)(round_up(rows, tile_m) / tile_m) * per_row, resident) ==
         rounds((uint64_t)(round_up(base, tile_m) / tile_m) * per_row, resident);
}

WsLayout make_layout(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank, bool routed,
                     bool pad_groups = false) {
  WsLayout w{};
  w.K_pad = k_padded(k);
  w.KB = w.K_pad / 32u;
  w.rows_bound = pad_groups ? padded_rows_bound(m, n_groups) : round_up(m, 32u);
  w.slots = round_up(w.rows_bound, kTileM);
  (void)routed;
  w.nkk = rank_chunks(rank);
  w.n_steps = (k + 63u) / 64u;
  w.steps_per_wave = (w.n_steps + 15u) / 16u;
  uint64_t off = 0;
  // The LoRA operands a caller may vouch for (MI355_W8A8_FLAG_LORA_PACK_VALID) come first: their sizes and
  // so their places depend on (k, n, n_adapters, rank) only -- not on m, the path or the slot layout -- so
  // calls of different row counts on one workspace find them where an earlier call left them.
  w.at = off; off += rank ? align256((uint64_t)n_groups * w.KB * w.nkk * kBlockBytes) : 0u;  // A in operand order
  w.bp = off; off += rank ? align256((uint64_t)n_groups * (n_padded(n) / 32u) * w.nkk * kBlockBytes) : 0u;
  w.xq = off; off += align256((uint64_t)w.slots * w.K_pad);
  w.sx = off; off += align256((uint64_t)w.slots * 4u);
  w.src_row = off; off += align256((uint64_t)w.slots * 4u);
  w.dst_pos = off; off += align256((uint64_t)m * 4u);
  w.slot_group = off; off += align256((uint64_t)w.slots * 4u);
  w.blk_range = off; off += align256((uint64_t)(w.slots / 32u) * 4u);
  w.tile_ctr = off; off += 1024u;  // two sets of eight counters, 64 bytes apart
  // normalized rows: only the decode path keeps them in memory (RMSNorm + LoRA, M <= 32)
  w.xn = off;
  off += (rank && m <= kSkinnyChunkedMaxRows) ? align256((uint64_t)(m < 32u ? m : 32u) * k * 2u) : 0u;
  w.zp = off; off += rank ? align256((uint64_t)(w.slots / 32u) * w.nkk * 3u * kBlockBytes) : 0u;
  w.skinny = off; off += align256(skinny_workspace_bytes(m, n, rank));
  w.total = off;
  return w;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool overlaps(const void* a, uint64_t an, const void* b, uint64_t bn) {
  if (!a || !b || an == 0 || bn == 0) return false;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + bn && b0 < a0 + an;
}

inline int launch_status() { return hipGetLastError() == hipSuccess ? MI355_W8A8_OK : MI355_W8A8_ERR_LAUNCH; }

template <bool RMS>
int launch_quant(const QuantArgs& a, hipStream_t s) {
  const uint32_t need = (a.K_pad + 511u) / 512u;
  const dim3 grid((a.M + 3u) / 4u), block(256);
#define W8A8_Q(NCH)                                                              \
  if (need <= NCH) {                                                             \
    hipLaunchKernelGGL((quant_rows_kernel<NCH, RMS>), grid, block, 0, s, a);     \
    return launch_status();                                                      \
  }
  W8A8_Q(1) W8A8_Q(2) W8A8_Q(4) W8A8_Q(8) W8A8_Q(16) W8A8_Q(24) W8A8_Q(32)
#undef W8A8_Q
  return MI355_W8A8_ERR_UNSUPPORTED;
}

// LoRA-A projection on the transposed A.  Up to 32 ranks the operands travel through LDS in whole
// cache lines (the staged form of the kernel); beyond, two rank blocks per wave leave no room for that.
int launch_lora_a(const LoraAArgs& la, uint32_t nkk, dim3 grid, hipStream_t s) {
  if (nkk > 2u) {
    hipLaunchKernelGGL((lora_a_kernel<2>), grid, dim3(1024), 0, s, la);
    return launch_status();
  }
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(&lora_a_kernel<1, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLoraAStageBytes) != hipSuccess)
    return MI355_W8A8_ERR_LAUNCH;
  hipLaunchKernelGGL((lora_a_kernel<1, true>), grid, dim3(1024), kLoraAStageBytes, s, la);
  return launch_status();
}

template <int EPI, int NKK, int MODE>
int launch_gemm_one(const GemmArgs& g, hipStream_t s) {
  // persistent grid: one workgroup slot per CU (two in the 256 x 128 geometry), a multiple of 8
  const uint32_t ntile = g.tiles_m * g.tiles_n;
  const uint32_t slots = (MODE == kModeDense || MODE == kModeDense128) ? 512u : 256u;
  const uint32_t want = ((ntile + 7u) / 8u) * 8u;
  const dim3 grid(want < slots ? want : slots), block(MODE == kModeGrouped128 ? 512 : 256);
  constexpr uint32_t lds_bytes =
      MODE == kModeGrouped128 ? kGrouped128LdsBytes
                              : (MODE == kModeGrouped ? kGroupedLdsBytes
                                                      : (MODE == kModeDense128 ? kGemmStages * kGemm128StageBytes : kGemmLdsBytes));
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(&w8a8_gemm_kernel<EPI, NKK, MODE>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
    return MI355_W8A8_ERR_LAUNCH;
  hipLaunchKernelGGL((w8a8_gemm_kernel<EPI, NKK, MODE>), grid, block, lds_bytes, s, g);
  return launch_status();
}

template <int EPI, int MODE = kModeDense>
int launch_gemm(const GemmArgs& g, uint32_t nkk, hipStream_t s) {
  switch (nkk) {
    case 0: return launch_gemm_one<EPI, 0, MODE>(g, s);
    case 1: return launch_gemm_one<EPI, 1, MODE>(g, s);
    case 2: return launch_gemm_one<EPI, 2, MODE>(g, s);
    case 4: return launch_gemm_one<EPI, 4, MODE>(g, s);
    default: return MI355_W8A8_ERR_UNSUPPORTED;
  }
}

template <int EPI, int NKK, int NW = 4>
int launch_gemm16_one(const GemmArgs& g, hipStream_t s) {
  // persistent grid: one workgroup per CU (two in the 256 x 128 geometry), a multiple of 8 so that every
  // XCD gets the same share
  using Geo = G16Geo<NW>;
  const uint32_t ntile = g.tiles_m * g.tiles_n;
  const uint32_t want = ((ntile + 7u) / 8u) * 8u;
  const dim3 grid(want < (uint32_t)Geo::kResident ? want : (uint32_t)Geo::kResident), block(Geo::kThreads);
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(&w8a8_gemm16_kernel<EPI, NKK, NW>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, Geo::kLdsBytes) != hipSuccess)
    return MI355_W8A8_ERR_LAUNCH;
  hipLaunchKernelGGL((w8a8_gemm16_kernel<EPI, NKK, NW>), grid, block, Geo::kLdsBytes, s, g);
  return launch_status();
}

template <int EPI, int NW = 4>
int launch_gemm16(const GemmArgs& g, uint32_t nkk, hipStream_t s) {
  switch (nkk) {
    case 0: return launch_gemm16_one<EPI, 0, NW>(g, s);
    case 1: return launch_gemm16_one<EPI, 1, NW>(g, s);
    case 2: return launch_gemm16_one<EPI, 2, NW>(g, s);
    case 4: return launch_gemm16_one<EPI, 4, NW>(g, s);
    default: return MI355_W8A8_ERR_UNSUPPORTED;
  }
}

int validate_common(uint32_t m, uint32_t k, uint32_t n) {
  if (m == 0 || k == 0 || n == 0) return MI355_W8A8_ERR_SHAPE;
  if (m > kMaxRows || n > kMaxN) return MI355_W8A8_ERR_UNSUPPORTED;
  if (k % 8u) return MI355_W8A8_ERR_UNSUPPORTED;
  if (k_padded(k) > kMaxK) return MI355_W8A8_ERR_UNSUPPORTED;
  if ((uint64_t)m * n >= (1ull << 32) - (1ull << 20)) return MI355_W8A8_ERR_UNSUPPORTED;  // 32-bit offsets
  return MI355_W8A8_OK;
}

// Skinny-M path: quantize -> stream (weight + LoRA-A units) -> epilogue.
int launch_skinny(const mi355_w8a8_problem* p, unsigned char* xq, float* sx, uint16_t* xn, unsigned char* sws,
                  uint32_t K_pad, uint32_t KB, hipStream_t s, bool allow_regroup = true) {
  const bool rms = p->rms_gamma != nullptr;
  const bool lora = p->n_adapters > 0;
  const SkinnyLayout L = skinny_layout(p->m, p->k, p->n, p->rank);
  int st;
  if (!(p->flags & MI355_W8A8_FLAG_SKIP_PROLOGUE)) {
    SkinnyQuantArgs q{};
    q.x = static_cast<const uint16_t*>(p->x);
    q.gamma = p->rms_gamma;
    q.eps = p->rms_eps;
    q.M = p->m; q.K = p->k; q.K_pad = K_pad; q.KB = KB;
    q.xq = xq; q.sx = sx;
    q.codes_rm = p->aux_x_codes; q.scales_rm = p->aux_x_scales;
    q.xn = (rms && lora) ? xn : nullptr;
    q.xn_aux = static_cast<uint16_t*>(p->aux_normalized);
    // without RMSNorm the LoRA-A units depend on x only and ride along with the quantizer
    q.lora_a = static_cast<const uint16_t*>(p->lora_a);
    q.idx = p->adapter_indices;
    q.z_part = reinterpret_cast<float*>(sws + L.z_part);
    q.n_adapters = p->n_adapters; q.r = p->rank; q.z_chunks = L.z_chunks; q.z_chunk_k = L.z_chunk_k;
    q.n_z_units = (lora && !rms) ? p->m * L.z_chunks : 0u;
    const bool regroup = allow_regroup && lora && p->rank <= 32u && p->m <= 16u && (p->n % 8u) == 0;
    // the caller may vouch that the regrouped B of an earlier call (same B, same adapter per row) is still
    // in the workspace; a call in 32-row chunks shares one workspace between its chunks and never keeps it
    const bool keep_regrouped = regroup && (p->flags & MI355_W8A8_FLAG_LORA_PACK_VALID);
    q.lora_b = (regroup && !keep_regrouped) ? static_cast<const uint16_t*>(p->lora_b) : nullptr;
    q.bsel = reinterpret_cast<uint16_t*>(sws + L.bsel);
    q.N = p->n; q.n_groups = n_padded(p->n) / 128u;
    q.lora_scaling = lora ? p->lora_scaling : nullptr;
    q.row_scaling = reinterpret_cast<float*>(sws + L.row_scaling);
    const uint32_t n_regroup = (regroup && !keep_regrouped) ? (p->m * q.n_groups + 3u) / 4u : 0u;
    if (rms) hipLaunchKernelGGL((skinny_quant_kernel<true>), dim3(p->m + n_regroup), dim3(1024), 0, s, q);
    else hipLaunchKernelGGL((skinny_quant_kernel<false>), dim3(p->m + q.n_z_units + n_regroup), dim3(1024), 0, s, q);
    if ((st = launch_status())) return st;
    if (lora && rms) {  // the LoRA-A units read the normalized rows the quantizer has just written
      SkinnyLoraAArgs la{};
      la.xsrc = xn; la.lora_a = static_cast<const uint16_t*>(p->lora_a); la.idx = p->adapter_indices;
      la.z_part = q.z_part; la.K = p->k; la.n_adapters = p->n_adapters; la.r = p->rank;
      la.z_chunks = L.z_chunks; la.z_chunk_k = L.z_chunk_k;
      hipLaunchKernelGGL(skinny_lora_a_kernel, dim3(p->m * L.z_chunks), dim3(1024), 0, s, la);
      if ((st = launch_status())) return st;
    }
  }
  if (p->flags & MI355_W8A8_FLAG_SKIP_GEMM) return MI355_W8A8_OK;
  SkinnyStreamArgs a{};
  a.xq = xq;
  a.wp = static_cast<const unsigned char*>(p->w_packed);
  a.z_part = reinterpret_cast<const float*>(sws + L.z_part);
  a.sx = sx; a.sw = p->w_scales;
  a.lora_b = lora ? static_cast<const uint16_t*>(p->lora_b) : nullptr;
  a.bsel = (allow_regroup && lora && p->rank <= 32u && p->m <= 16u && (p->n % 8u) == 0)
               ? reinterpret_cast<const uint16_t*>(sws + L.bsel) : nullptr;
  a.lora_scaling = p->lora_scaling; a.idx = p->adapter_indices;
  a.row_scaling = reinterpret_cast<const float*>(sws + L.row_scaling);
  a.residual = static_cast<const uint16_t*>(p->residual);
  a.out = static_cast<uint16_t*>(p->out);
  a.aux_acc = p->aux_acc;
  a.M = p->m; a.N = p->n; a.N_pad = n_padded(p->n); a.K = p->k; a.KB = KB;
  a.pairs_per_wave = L.pairs_per_wave;
  a.n_adapters = p->n_adapters; a.r = p->rank; a.z_chunks = L.z_chunks;
  a.n_groups = a.N_pad / 128u;
  // eight units per 128-column group; groups are dealt to the eight XCD residues of the block index
  const dim3 grid(((a.n_groups + 7u) / 8u) * 64u), block(kSkinnyStreamThreads);
  if (p->m > 16u) hipLaunchKernelGGL((skinny_stream_kernel<true>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((skinny_stream_kernel<false>), grid, block, 0, s, a);
  return launch_status();
}

enum Required { kReqNone = 0, kReqLinear = 1, kReqGateUp = 2, kReqResidual = 3 };

// Which kernels a forward call of these dimensions runs (an MI355_W8A8_PATH_* value), or a negative
// status for a contradictory request.  The choice depends on the dimensions and the flags only.
int choose_forward_path(uint32_t m, uint32_t k, uint32_t n, uint32_t flags) {
  const bool swiglu = (flags & MI355_W8A8_FLAG_SWIGLU) != 0;
  bool skinny = m <= (uint32_t)kSkinnyMaxRows && !(flags & MI355_W8A8_FLAG_FORCE_TILED) && !swiglu;
  if (flags & MI355_W8A8_FLAG_FORCE_SKINNY) {
    if (m > (uint32_t)kSkinnyMaxRows || swiglu) return MI355_W8A8_ERR_UNSUPPORTED;
    skinny = true;
  }
  if (!skinny_supported()) skinny = false;
  if (skinny) return MI355_W8A8_PATH_SKINNY;
  if (skinny_supported() && !swiglu && skinny_chunked_pays(m, k, n) &&
      !(flags & (MI355_W8A8_FLAG_FORCE_TILED | MI355_W8A8_FLAG_TILE_256X128 | MI355_W8A8_FLAG_TILE_256X256 |
                 MI355_W8A8_FLAG_TILE_128X128 | MI355_W8A8_FLAG_TILE_256X128_PAIR)))
    return MI355_W8A8_PATH_SKINNY_CHUNKS;
  // 256 x 256 tiles (one 8-wave workgroup per CU, 16 x 16 x 64 MFMAs) once they fill half the CUs;
  // below that the 256 x 128 geometry (two 4-wave workgroups per CU) has twice the tiles to spread.
  // Measured on the Qwen3-4B QKV projection (K = 2560, N = 6144, rank-64 adapters): at 192 tiles
  // (M = 2048) the GEMM takes 55 us against 73 us; at 48-80 tiles the two are level.
  bool wide = (uint64_t)(round_up(m, kTileM) / kTileM) * (n_padded(n) / kG16TileN) >= 128u;
  if (flags & MI355_W8A8_FLAG_TILE_256X128) wide = false;
  if (flags & MI355_W8A8_FLAG_TILE_256X256) wide = true;
  if (k_padded(k) < kG16MinKPad) wide = false;  // its stage schedule needs at least six 64-wide k steps
  // 128 x 128 tiles (32 x 128 per wave) while all of them are resident at once (two workgroups per
  // CU): a wave then carries half the MFMAs and half the epilogue of the 256 x 128 geometry and the
  // call spreads over four times the CUs.  Measured (call, rank-64 adapters): K = 2560, N = 6144 at
  // M = 512: 62 us against 84; K = 4096, N = 2560 at M = 2048: 88 against 105; beyond 512 tiles the
  // larger geometries win (K = 2560, N = 6144 at M = 2048: 97 us against 85 on 256 x 256).
  const bool small = (uint64_t)(round_up(m, (uint32_t)kGemm128TileM) / (uint32_t)kGemm128TileM) * (n_padded(n) / kGemmTileN) <= 512u;
  const uint32_t forced = flags & (MI355_W8A8_FLAG_TILE_256X128 | MI355_W8A8_FLAG_TILE_256X256 | MI355_W8A8_FLAG_TILE_128X128 |
                                   MI355_W8A8_FLAG_TILE_256X128_PAIR);
  if (forced & (forced - 1u)) return MI355_W8A8_ERR_SHAPE;  // two geometries asked for
  if (forced == MI355_W8A8_FLAG_TILE_256X128_PAIR)  // (its stage schedule needs at least six 64-wide k steps, too)
    return k_padded(k) < kG16MinKPad ? MI355_W8A8_PATH_TILED_256X128 : MI355_W8A8_PATH_TILED_256X128_PAIR;
  if (forced == MI355_W8A8_FLAG_TILE_128X128 || (!forced && small)) return MI355_W8A8_PATH_TILED_128X128;
  return wide ? MI355_W8A8_PATH_TILED_256X256 : MI355_W8A8_PATH_TILED_256X128;
}

int run_forward(const mi355_w8a8_problem* p, hipStream_t s, Required req) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_problem)) return MI355_W8A8_ERR_STRUCT;
  int st = validate_common(p->m, p->k, p->n);
  if (st) return st;
  if (!p->x || !p->w_packed || !p->w_scales || !p->out) return MI355_W8A8_ERR_NULL;
  const bool swiglu = (p->flags & MI355_W8A8_FLAG_SWIGLU) != 0;
  const bool rms = p->rms_gamma != nullptr;
  const bool lora = p->n_adapters > 0;
  if (req == kReqLinear && (swiglu || rms || p->residual)) return MI355_W8A8_ERR_SHAPE;
  if (req == kReqGateUp && (!swiglu || !rms)) return MI355_W8A8_ERR_SHAPE;
  if (req == kReqResidual && (!p->residual || swiglu)) return MI355_W8A8_ERR_SHAPE;
  if (swiglu && (p->n & 1u)) return MI355_W8A8_ERR_SHAPE;
  if (swiglu && p->residual) return MI355_W8A8_ERR_UNSUPPORTED;
  if ((p->flags & MI355_W8A8_FLAG_FORCE_TILED) && (p->flags & MI355_W8A8_FLAG_FORCE_SKINNY))
    return MI355_W8A8_ERR_SHAPE;
  if (lora) {
    if (!p->lora_a || !p->lora_b || !p->lora_scaling) return MI355_W8A8_ERR_NULL;
    if (p->rank == 0 || p->rank > (uint32_t)kMaxRank) return MI355_W8A8_ERR_UNSUPPORTED;
    if (p->n_adapters > (uint32_t)kMaxAdapters) return MI355_W8A8_ERR_UNSUPPORTED;
  } else if (p->adapter_indices) {
    return MI355_W8A8_ERR_SHAPE;
  }
  if (p->aux_normalized && !rms) return MI355_W8A8_ERR_SHAPE;
  const uint32_t n_out = swiglu ? p->n / 2u : p->n;
  const uint64_t out_bytes = (uint64_t)p->m * n_out * 2u;
  const uint64_t x_bytes = (uint64_t)p->m * p->k * 2u;
  if (!aligned16(p->x) || !aligned16(p->w_packed) || !aligned16(p->out) || !aligned16(p->w_scales) ||
      !aligned16(p->lora_a) || !aligned16(p->lora_b) || !aligned16(p->residual) ||
      !aligned16(p->rms_gamma) || !aligned16(p->adapter_indices))
    return MI355_W8A8_ERR_ALIGN;
  if (overlaps(p->out, out_bytes, p->x, x_bytes) || overlaps(p->out, out_bytes, p->residual, out_bytes) ||
      overlaps(p->out, out_bytes, p->w_packed, mi355_w8a8_packed_weight_bytes(p->k, p->n)) ||
      overlaps(p->out, out_bytes, p->lora_b, (uint64_t)p->n_adapters * p->rank * p->n * 2u) ||
      overlaps(p->out, out_bytes, p->lora_a, (uint64_t)p->n_adapters * p->rank * p->k * 2u) ||
      overlaps(p->out, out_bytes, p->workspace, p->workspace_bytes))
    return MI355_W8A8_ERR_ALIAS;

  const bool routed = lora && p->adapter_indices && p->n_adapters > 1;
  // The workspace is always sized for the routed layout so one allocation serves every call.
  const uint64_t need = mi355_w8a8_workspace_bytes(p->m, p->k, p->n, p->n_adapters, p->rank, p->flags);
  if (!p->workspace) return MI355_W8A8_ERR_WORKSPACE;
  if (p->workspace_bytes < need) return MI355_W8A8_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return MI355_W8A8_ERR_ALIGN;
  const int path = choose_forward_path(p->m, p->k, p->n, p->flags);
  if (path < 0) return path;
  // groups on block boundaries: only where the quantizer sorts the rows itself and the tiles stay resident
  const bool pad_groups =
      routed && ((path == MI355_W8A8_PATH_TILED_128X128 && padded_groups_fit(p->m, p->n, p->n_adapters)) ||
                 (path == MI355_W8A8_PATH_TILED_256X256 && padded_groups_fit(p->m, p->n, p->n_adapters, true)));
  const WsLayout w = make_layout(p->m, p->k, p->n, p->n_adapters, lora ? p->rank : 0u, routed, pad_groups);
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  int32_t* src_row = reinterpret_cast<int32_t*>(ws + w.src_row);
  int32_t* dst_pos = reinterpret_cast<int32_t*>(ws + w.dst_pos);
  int32_t* slot_group = reinterpret_cast<int32_t*>(ws + w.slot_group);
  int32_t* blk_range = reinterpret_cast<int32_t*>(ws + w.blk_range);

  (void)hipGetLastError();  // drop a stale error so it is not blamed on these launches

  const bool skinny = path == MI355_W8A8_PATH_SKINNY;
  if (skinny) {
    return launch_skinny(p, ws + w.xq, reinterpret_cast<float*>(ws + w.sx),
                         reinterpret_cast<uint16_t*>(ws + w.xn), ws + w.skinny, w.K_pad, w.KB, s);
  }
  if (path == MI355_W8A8_PATH_SKINNY_CHUNKS) {
    // The chunks overwrite each other's prologue results, so there is no GEMM-only or prologue-only
    // rerun of such a call; the choice of path must not depend on those flags either (a GEMM-only
    // tiled call would read tables no tiled prologue has written).
    if (p->flags & (MI355_W8A8_FLAG_SKIP_PROLOGUE | MI355_W8A8_FLAG_SKIP_GEMM)) return MI355_W8A8_ERR_UNSUPPORTED;
    for (uint32_t row0 = 0; row0 < p->m; row0 += (uint32_t)kSkinnyMaxRows) {
      mi355_w8a8_problem sub = *p;
      sub.m = p->m - row0 < (uint32_t)kSkinnyMaxRows ? p->m - row0 : (uint32_t)kSkinnyMaxRows;
      sub.x = static_cast<const unsigned char*>(p->x) + (size_t)row0 * p->k * 2u;
      sub.out = static_cast<unsigned char*>(p->out) + (size_t)row0 * p->n * 2u;
      if (p->residual) sub.residual = static_cast<const unsigned char*>(p->residual) + (size_t)row0 * p->n * 2u;
      if (p->adapter_indices) sub.adapter_indices = p->adapter_indices + row0;
      if (p->aux_x_codes) sub.aux_x_codes = p->aux_x_codes + (size_t)row0 * p->k;
      if (p->aux_x_scales) sub.aux_x_scales = p->aux_x_scales + row0;
      if (p->aux_acc) sub.aux_acc = p->aux_acc + (size_t)row0 * p->n;
      if (p->aux_normalized)
        sub.aux_normalized = static_cast<unsigned char*>(p->aux_normalized) + (size_t)row0 * p->k * 2u;
      // the chunks share the workspace: they run one after the other on the stream
      if ((st = launch_skinny(&sub, ws + w.xq, reinterpret_cast<float*>(ws + w.sx),
                              reinterpret_cast<uint16_t*>(ws + w.xn), ws + w.skinny, w.K_pad, w.KB, s, false)))
        return st;
    }
    return MI355_W8A8_OK;
  }

  const bool skip_prologue = (p->flags & MI355_W8A8_FLAG_SKIP_PROLOGUE) != 0;
  const bool skip_gemm = (p->flags & MI355_W8A8_FLAG_SKIP_GEMM) != 0;
  // Up to 8192 rows the quantizer's workgroups sort the adapter indices themselves (one launch less) --
  // unless the launch that lays out the LoRA operands runs anyway (adapters that changed since the last
  // call, as in every training step): then its first block sorts, beside the others, and the quantizer
  // reads the tables (4-6 us less in each of its workgroups).
  const bool pack_launch = lora && !skip_prologue && !(p->flags & MI355_W8A8_FLAG_LORA_PACK_VALID);
  const bool route_inline = routed && p->m <= kInlineRouteMaxRows && !pack_launch;
  if ((routed || lora) && !skip_prologue) {
    LoraPrepArgs pa{};
    pa.idx = routed ? p->adapter_indices : nullptr;
    pa.src_row = src_row; pa.dst_pos = dst_pos; pa.slot_group = slot_group; pa.blk_range = blk_range;
    pa.lora_a = static_cast<const uint16_t*>(p->lora_a);
    pa.lora_b = static_cast<const uint16_t*>(p->lora_b);
    pa.at = reinterpret_cast<uint16_t*>(ws + w.at);
    pa.bp = ws + w.bp;
    pa.M = p->m; pa.K = p->k; pa.N = p->n; pa.n_groups = p->n_adapters; pa.r = p->rank; pa.nkk = w.nkk;
    pa.ncb = n_padded(p->n) / 32u; pa.slots = w.slots;
    pa.route_blocks = (routed && !route_inline) ? 1u : 0u;
    pa.route_pad = pad_groups ? 32u : 1u;
    pa.a_operand_kb = w.KB;  // the quantizer reads A in MFMA operand order
    const uint64_t a_items = (uint64_t)p->n_adapters * w.KB * w.nkk * 64u;
    const uint64_t b_items = (uint64_t)p->n_adapters * pa.ncb * w.nkk * 64u;
    const bool pack = !(p->flags & MI355_W8A8_FLAG_LORA_PACK_VALID);  // else the workspace holds both already
    pa.a_blocks = pack ? (uint32_t)((a_items + 1023u) / 1024u) : 0u;
    const uint32_t b_blocks = pack ? (uint32_t)((b_items + 1023u) / 1024u) : 0u;
    if (pa.route_blocks + pa.a_blocks + b_blocks) {
      hipLaunchKernelGGL(lora_prep_kernel, dim3(pa.route_blocks + pa.a_blocks + b_blocks), dim3(1024), 0, s, pa);
      if ((st = launch_status())) return st;
    }
  }

  // quantizer and LoRA-A projection: one pass over x
  QuantLoraArgs q{};
  q.x = static_cast<const uint16_t*>(p->x);
  q.gamma = p->rms_gamma;
  q.eps = p->rms_eps;
  q.M = p->m; q.K = p->k; q.K_pad = w.K_pad; q.KB = w.KB;
  q.n_half_blocks = w.rows_bound / 16u;
  q.src_row = routed ? src_row : nullptr;
  q.slot_group = routed ? slot_group : nullptr;
  q.blk_range = routed ? blk_range : nullptr;
  q.xq_packed = ws + w.xq;
  q.sx_slots = reinterpret_cast<float*>(ws + w.sx);
  q.codes_rm = p->aux_x_codes;
  q.scales_rm = p->aux_x_scales;
  q.xn_aux = static_cast<uint16_t*>(p->aux_normalized);
  q.at = lora ? reinterpret_cast<const uint16_t*>(ws + w.at) : nullptr;
  q.zp = ws + w.zp;
  q.r = p->rank; q.nkk = w.nkk;
  q.nterms = (p->flags & MI355_W8A8_FLAG_LORA_SPLIT2) ? 2u : 3u;
  q.tile_ctr = reinterpret_cast<uint32_t*>(ws + w.tile_ctr);
  q.group_pad = pad_groups ? 32u : 1u;
  q.rows_per_wg = quant_lora_rows_per_wg(p->k);
  q.row_stride = quant_lora_row_stride(p->k);
  if (route_inline) {
    q.route_idx = p->adapter_indices; q.n_groups = p->n_adapters; q.slots = w.slots;
    q.src_row = src_row; q.slot_group = slot_group; q.blk_range = blk_range;
  }
  if (!skip_prologue) {
    const dim3 grid(q.n_half_blocks * (16u / q.rows_per_wg)), block(1024);
    const uint32_t ql_lds = quant_lora_lds_bytes(p->k, lora ? w.nkk : 0u);
#define W8A8_QL1(CB, RMS)                                                                                   \
  {                                                                                                         \
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&quant_lora_kernel<CB, RMS>),                     \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)ql_lds) != hipSuccess)         \
      return MI355_W8A8_ERR_LAUNCH;                                                                         \
    hipLaunchKernelGGL((quant_lora_kernel<CB, RMS>), grid, block, ql_lds, s, q);                            \
  }
#define W8A8_QL(CB)                \
  if (rms) W8A8_QL1(CB, true)      \
  else W8A8_QL1(CB, false)
    switch (lora ? w.nkk : 0u) {
      case 0: W8A8_QL(0); break;
      case 1: W8A8_QL(1); break;
      case 2: W8A8_QL(2); break;
      default: W8A8_QL(4); break;
    }
#undef W8A8_QL
#undef W8A8_QL1
    if ((st = launch_status())) return st;
  } else if (!skip_gemm && path != MI355_W8A8_PATH_TILED_256X256) {
    // measurement calls: the tile counters of the 256 x 128 geometry's dynamic schedule still have to
    // start at zero (the 256 x 256 kernel has a static schedule and no counters)
    hipLaunchKernelGGL(zero_words_kernel, dim3(1), dim3(256), 0, s, q.tile_ctr, 256u);
    if ((st = launch_status())) return st;
  }

  if (skip_gemm) return MI355_W8A8_OK;
  GemmArgs g{};
  g.xq = ws + w.xq;
  g.wp = static_cast<const unsigned char*>(p->w_packed);
  g.sx = reinterpret_cast<const float*>(ws + w.sx);
  g.sw = p->w_scales;
  g.zp = lora ? ws + w.zp : nullptr;
  g.bp = lora ? ws + w.bp : nullptr;
  g.lora_scaling = p->lora_scaling;
  g.src_row = routed ? src_row : nullptr;
  g.slot_group = routed ? slot_group : nullptr;
  g.blk_range = routed ? blk_range : nullptr;
  g.residual = static_cast<const uint16_t*>(p->residual);
  g.out = p->out;
  g.M = p->m; g.N = p->n; g.K_pad = w.K_pad; g.KB = w.KB; g.slots = w.slots;
  g.total_rows = w.rows_bound;
  g.groups_per_weight = 1;
  g.tiles_m = w.slots / kTileM;
  g.tiles_n = n_padded(p->n) / kGemmTileN;
  g.rank = lora ? p->rank : 0u;
  g.tile_ctr = reinterpret_cast<uint32_t*>(ws + w.tile_ctr);
  const bool wide = path == MI355_W8A8_PATH_TILED_256X256;
  const bool pair = path == MI355_W8A8_PATH_TILED_256X128_PAIR;
  const bool small = path == MI355_W8A8_PATH_TILED_128X128;
  if (wide) g.tiles_n = n_padded(p->n) / kG16TileN;
  if (small) g.tiles_m = round_up(w.rows_bound, (uint32_t)kGemm128TileM) / (uint32_t)kGemm128TileM;
  if (p->aux_acc) {
    GemmArgs ga = g;
    ga.out = p->aux_acc;
    ga.residual = nullptr;
    if ((st = wide ? launch_gemm16_one<kEpiAcc, 0>(ga, s)
                   : (pair ? launch_gemm16_one<kEpiAcc, 0, 2>(ga, s)
                           : (small ? launch_gemm<kEpiAcc, kModeDense128>(ga, 0u, s) : launch_gemm<kEpiAcc>(ga, 0u, s)))))
      return st;
    g.tile_ctr += 128;  // the second counter set
  }
  if (wide) return swiglu ? launch_gemm16<kEpiSwiglu>(g, w.nkk, s) : launch_gemm16<kEpiPlain>(g, w.nkk, s);
  if (pair) return swiglu ? launch_gemm16<kEpiSwiglu, 2>(g, w.nkk, s) : launch_gemm16<kEpiPlain, 2>(g, w.nkk, s);
  if (small)
    return swiglu ? launch_gemm<kEpiSwiglu, kModeDense128>(g, w.nkk, s) : launch_gemm<kEpiPlain, kModeDense128>(g, w.nkk, s);
  return swiglu ? launch_gemm<kEpiSwiglu>(g, w.nkk, s) : launch_gemm<kEpiPlain>(g, w.nkk, s);
}

struct GroupedLayout {
  uint64_t xq, sx, zp, at, bp, src_row, dst_pos, blk_range, total;
  uint32_t slots, nkk, K_pad, KB, n_steps, steps_per_wave, pad;
};

// Rows of padding per group = rows of a GEMM tile: 128 once the groups average at least 96 rows (the
// weight panel then travels L2 -> LDS once per 128 rows), else 64; the flags force either.
uint32_t grouped_pad(uint32_t m, uint32_t n_groups, uint32_t flags) {
  if (flags & MI355_W8A8_FLAG_GROUPED_TILE64) return 64u;
  if (flags & MI355_W8A8_FLAG_GROUPED_TILE128) return 128u;
  return (uint64_t)m >= 96ull * n_groups ? 128u : 64u;
}

GroupedLayout make_grouped_layout(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank,
                                  uint32_t flags) {
  GroupedLayout w{};
  w.K_pad = k_padded(k);
  w.KB = w.K_pad / 32u;
  w.pad = grouped_pad(m, n_groups, flags);
  // every group is padded to a multiple of pad slots: at most pad - 1 padding slots per group
  const uint64_t worst = (uint64_t)m + (uint64_t)(w.pad - 1u) * n_groups;
  w.slots = (uint32_t)((worst + w.pad - 1u) / w.pad * w.pad);
  w.nkk = rank_chunks(rank);
  w.n_steps = (k + 63u) / 64u;
  w.steps_per_wave = (w.n_steps + 15u) / 16u;
  uint64_t off = 0;
  // (the LoRA operands a caller may vouch for come first, as in make_layout: their places depend on
  // (k, n, n_groups, rank) only, not on the row count)
  w.at = off; off += rank ? align256((uint64_t)n_groups * rank * k * 2u) : 0u;
  w.bp = off; off += rank ? align256((uint64_t)n_groups * (n_padded(n) / 32u) * w.nkk * kBlockBytes) : 0u;
  w.xq = off; off += align256((uint64_t)w.slots * w.K_pad);
  w.sx = off; off += align256((uint64_t)w.slots * 4u);
  w.src_row = off; off += align256((uint64_t)w.slots * 4u);
  w.dst_pos = off; off += align256((uint64_t)m * 4u);
  w.blk_range = off; off += align256((uint64_t)(w.slots / 32u) * 4u);
  w.zp = off; off += rank ? align256((uint64_t)(w.slots / 32u) * w.nkk * 3u * kBlockBytes) : 0u;
  w.total = off;
  return w;
}

int run_grouped(const mi355_w8a8_grouped_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_grouped_problem)) return MI355_W8A8_ERR_STRUCT;
  int st = validate_common(p->m, p->k, p->n);
  if (st) return st;
  if (p->n_groups == 0) return MI355_W8A8_ERR_SHAPE;
  if (p->n_groups > (uint32_t)kMaxGroups) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!p->x || !p->w_packed || !p->w_scales || !p->out || !p->group_sizes) return MI355_W8A8_ERR_NULL;
  const bool swiglu = (p->flags & MI355_W8A8_FLAG_SWIGLU) != 0;
  if (swiglu && (p->n & 1u)) return MI355_W8A8_ERR_SHAPE;
  const bool lora = p->rank > 0;
  if (lora) {
    if (!p->lora_a || !p->lora_b || !p->lora_scaling) return MI355_W8A8_ERR_NULL;
    if (p->rank > (uint32_t)kMaxRank) return MI355_W8A8_ERR_UNSUPPORTED;
  }
  const uint32_t gpw = p->groups_per_weight ? p->groups_per_weight : 1u;
  if (p->n_groups % gpw) return MI355_W8A8_ERR_SHAPE;
  const uint32_t n_out = swiglu ? p->n / 2u : p->n;
  const uint64_t out_bytes = (uint64_t)p->m * n_out * 2u;
  if (!aligned16(p->x) || !aligned16(p->w_packed) || !aligned16(p->out) || !aligned16(p->w_scales) ||
      !aligned16(p->lora_a) || !aligned16(p->lora_b) || (reinterpret_cast<uintptr_t>(p->group_sizes) & 3u))
    return MI355_W8A8_ERR_ALIGN;
  const uint32_t x_repeat = p->x_row_map ? p->x_row_repeat : 1u;
  if (p->x_row_map && (x_repeat == 0 || (reinterpret_cast<uintptr_t>(p->x_row_map) & 3u)))
    return x_repeat == 0 ? MI355_W8A8_ERR_SHAPE : MI355_W8A8_ERR_ALIGN;
  // with a row map x holds one row per token unless the caller says otherwise; gathered reads are
  // clamped to these rows
  const uint32_t x_rows = (p->x_row_map && p->x_rows) ? p->x_rows : (p->m + x_repeat - 1u) / x_repeat;
  if (overlaps(p->out, out_bytes, p->x, (uint64_t)x_rows * p->k * 2u) ||
      overlaps(p->out, out_bytes, p->x_row_map, (uint64_t)p->m * 4u) ||
      overlaps(p->out, out_bytes, p->workspace, p->workspace_bytes))
    return MI355_W8A8_ERR_ALIAS;
  if ((p->flags & MI355_W8A8_FLAG_GROUPED_TILE64) && (p->flags & MI355_W8A8_FLAG_GROUPED_TILE128))
    return MI355_W8A8_ERR_SHAPE;
  const GroupedLayout w = make_grouped_layout(p->m, p->k, p->n, p->n_groups, p->rank, p->flags);
  if (!p->workspace || p->workspace_bytes < w.total) return MI355_W8A8_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return MI355_W8A8_ERR_ALIGN;
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  int32_t* src_row = reinterpret_cast<int32_t*>(ws + w.src_row);
  int32_t* dst_pos = reinterpret_cast<int32_t*>(ws + w.dst_pos);
  int32_t* blk_range = reinterpret_cast<int32_t*>(ws + w.blk_range);
  (void)hipGetLastError();

  // measurement only: a call with SKIP_PROLOGUE after a full call with the same arguments and workspace
  // re-runs only the GEMM kernel; SKIP_GEMM stops after routing / quantization / LoRA-A
  const bool skip_prologue = (p->flags & MI355_W8A8_FLAG_SKIP_PROLOGUE) != 0;
  const bool skip_gemm = (p->flags & MI355_W8A8_FLAG_SKIP_GEMM) != 0;
  if (skip_prologue && (p->aux_x_codes || p->aux_x_scales)) return MI355_W8A8_ERR_UNSUPPORTED;

  // launch 1: the slot layout of the groups next to the LoRA operand re-layouts
  if (!skip_prologue) {
    LoraPrepArgs pa{};
    pa.src_row = src_row; pa.dst_pos = dst_pos; pa.blk_range = blk_range;
    pa.group_sizes = p->group_sizes; pa.group_pad = w.pad;
    pa.lora_a = static_cast<const uint16_t*>(p->lora_a);
    pa.lora_b = static_cast<const uint16_t*>(p->lora_b);
    pa.at = reinterpret_cast<uint16_t*>(ws + w.at);
    pa.bp = ws + w.bp;
    pa.M = p->m; pa.K = p->k; pa.N = p->n; pa.n_groups = p->n_groups; pa.r = p->rank; pa.nkk = w.nkk;
    pa.ncb = n_padded(p->n) / 32u; pa.slots = w.slots;
    // (the layout is filled slot by slot: a few workgroups, each with the prefix sums of its own)
    pa.route_blocks = (w.slots + 2047u) / 2048u < 16u ? (w.slots + 2047u) / 2048u : 16u;
    uint32_t b_blocks = 0;
    // (a caller that vouches for the operand packs of an earlier call on this workspace keeps them: the
    // launch then only lays out the slots)
    if (lora && !(p->flags & MI355_W8A8_FLAG_LORA_PACK_VALID)) {
      const uint64_t a_items = (uint64_t)p->n_groups * p->k * ((p->rank + 7u) / 8u);
      const uint64_t b_items = (uint64_t)p->n_groups * pa.ncb * w.nkk * 64u;
      pa.a_blocks = (uint32_t)((a_items + 1023u) / 1024u);
      b_blocks = (uint32_t)((b_items + 1023u) / 1024u);
    }
    hipLaunchKernelGGL(lora_prep_kernel, dim3(pa.route_blocks + pa.a_blocks + b_blocks), dim3(1024), 0, s, pa);
    if ((st = launch_status())) return st;
  }

  // launch 2: the quantizer, a wave per row (measured faster here than the fused quantizer + LoRA-A
  // kernel of the dense path, whose 16-slot workgroups are sized for longer rows)
  if (!skip_prologue) {
  QuantArgs q{};
  q.x = static_cast<const uint16_t*>(p->x);
  q.M = p->m; q.K = p->k; q.K_pad = w.K_pad; q.KB = w.KB;
  q.dst_pos = dst_pos;
  q.xq_packed = ws + w.xq;
  q.sx_slots = reinterpret_cast<float*>(ws + w.sx);
  q.codes_rm = p->aux_x_codes;
  q.scales_rm = p->aux_x_scales;
  q.zero_out = static_cast<uint16_t*>(p->out);
  q.zero_cols = n_out;
  q.row_map = p->x_row_map; q.row_div = x_repeat; q.row_limit = x_rows;
  if ((st = launch_quant<false>(q, s))) return st;
  }

  // launch 3: LoRA-A projection per 32-slot block
  if (lora && !skip_prologue) {
    LoraAArgs la{};
    la.xsrc = static_cast<const uint16_t*>(p->x);
    la.at = reinterpret_cast<const uint16_t*>(ws + w.at);
    la.src_row = src_row;
    la.slot_group = nullptr;
    la.blk_range = blk_range;
    la.row_map = p->x_row_map; la.row_div = x_repeat; la.row_limit = x_rows;
    la.zp = ws + w.zp;
    la.M = p->m; la.K = p->k; la.r = p->rank; la.nkk = w.nkk;
    la.steps_per_wave = w.steps_per_wave; la.n_steps = w.n_steps;
    la.nterms = (p->flags & MI355_W8A8_FLAG_LORA_SPLIT2) ? 2u : 3u;
    la.n_blocks = w.slots / 32u;
    const dim3 grid(w.slots / 32u);
    if ((st = launch_lora_a(la, w.nkk, grid, s))) return st;
  }
  if (skip_gemm) return MI355_W8A8_OK;

  GemmArgs g{};
  g.xq = ws + w.xq;
  g.wp = static_cast<const unsigned char*>(p->w_packed);
  g.sx = reinterpret_cast<const float*>(ws + w.sx);
  g.sw = p->w_scales;
  g.zp = lora ? ws + w.zp : nullptr;
  g.bp = lora ? ws + w.bp : nullptr;
  g.lora_scaling = p->lora_scaling;
  g.src_row = src_row;
  g.slot_group = nullptr;
  g.blk_range = blk_range;
  g.residual = nullptr;
  g.out = p->out;
  g.w_group_stride = mi355_w8a8_packed_weight_bytes(p->k, p->n);
  g.M = p->m; g.N = p->n; g.K_pad = w.K_pad; g.KB = w.KB; g.slots = w.slots;
  g.total_rows = w.slots;
  g.tiles_m = w.slots / w.pad;
  g.tiles_n = (n_padded(p->n) + kGroupedTileN - 1u) / kGroupedTileN;
  g.rank = p->rank;
  g.groups_per_weight = gpw;
  if (p->aux_acc) {
    GemmArgs ga = g;
    ga.out = p->aux_acc;
    if ((st = w.pad == 128u ? launch_gemm<kEpiAcc, kModeGrouped128>(ga, 0u, s)
                            : launch_gemm<kEpiAcc, kModeGrouped>(ga, 0u, s)))
      return st;
  }
  if (w.pad == 128u)
    return swiglu ? launch_gemm<kEpiSwiglu, kModeGrouped128>(g, w.nkk, s)
                  : launch_gemm<kEpiPlain, kModeGrouped128>(g, w.nkk, s);
  return swiglu ? launch_gemm<kEpiSwiglu, kModeGrouped>(g, w.nkk, s) : launch_gemm<kEpiPlain, kModeGrouped>(g, w.nkk, s);
}

// ---------------------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------------------
struct BwdLayout {
  uint64_t dyp, swp, at, ap, rp, z, r_raw, rs, rpart, src_row, dst_pos, slot_group, blk_range, group_off, partA, partB, total;
  uint32_t slots, nkk, K_pad, KB, N_pad, NB, tiles_m, tiles_k, max_chunks, R, n_slices, groups_per_slice;
};

BwdLayout make_bwd_layout(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank) {
  BwdLayout w{};
  w.K_pad = k_padded(k); w.KB = w.K_pad / 32u;
  w.N_pad = n_padded(n); w.NB = w.N_pad / 32u;
  w.slots = round_up(m, kTileM);
  w.tiles_m = w.slots / 256u;
  w.tiles_k = (w.K_pad + 255u) / 256u;
  w.nkk = rank_chunks(rank);
  w.R = w.nkk > 2u ? 64u : 32u;  // rank rows of a partial (32-wide rank blocks)
  w.max_chunks = (m + kBwdChunkRows - 1u) / kBwdChunkRows + n_groups;
  {  // dy is packed (and r accumulated) by workgroups that own a slice of the 128-column groups
    const uint32_t ng = w.N_pad / 128u;
    w.n_slices = (ng + 3u) / 4u < 8u ? (ng + 3u) / 4u : 8u;
    w.groups_per_slice = (ng + w.n_slices - 1u) / w.n_slices;
  }
  uint64_t off = 0;
  w.dyp = off; off += align256((uint64_t)w.slots * w.N_pad * 2u);
  w.swp = off; off += align256((uint64_t)(w.N_pad + kBwdScalePad) * 4u);  // a stage fetches 1 KiB of scales starting at its own 32
  w.src_row = off; off += align256((uint64_t)w.slots * 4u);
  w.dst_pos = off; off += align256((uint64_t)m * 4u);
  w.slot_group = off; off += align256((uint64_t)w.slots * 4u);
  w.blk_range = off; off += align256((uint64_t)(w.slots / 32u) * 4u);
  w.group_off = off; off += align256((uint64_t)(kMaxAdapters + 1) * 4u);
  if (rank) {
    w.at = off; off += align256((uint64_t)n_groups * rank * k * 2u);
    w.ap = off; off += align256((uint64_t)n_groups * w.KB * w.nkk * kBlockBytes);
    w.rp = off; off += align256((uint64_t)(w.slots / 32u) * w.nkk * 3u * kBlockBytes);
    w.z = off; off += align256((uint64_t)w.slots * kBwdRankStride * 4u);
    w.r_raw = off; off += align256((uint64_t)w.slots * kBwdRankStride * 4u);
    w.rs = off; off += align256((uint64_t)w.slots * kBwdRankStride * 4u);
    w.rpart = off; off += align256((uint64_t)w.n_slices * w.slots * kBwdRankStride * 4u);  // also the K slices of z
    w.partA = off; off += align256((uint64_t)w.max_chunks * w.R * k * 4u);
    w.partB = off; off += align256((uint64_t)w.max_chunks * w.R * n * 4u);
  }
  w.total = off;
  return w;
}

int validate_bwd_dims(uint32_t m, uint32_t k, uint32_t n, uint32_t n_adapters, uint32_t rank) {
  int st = validate_common(m, k, n);
  if (st) return st;
  if (n % 8u) return MI355_W8A8_ERR_UNSUPPORTED;
  if ((uint64_t)m * k >= (1ull << 32) - (1ull << 20)) return MI355_W8A8_ERR_UNSUPPORTED;  // 32-bit offsets
  if (n_adapters > (uint32_t)kMaxAdapters || rank > (uint32_t)kMaxRank) return MI355_W8A8_ERR_UNSUPPORTED;
  if (n_adapters && rank == 0) return MI355_W8A8_ERR_UNSUPPORTED;
  return MI355_W8A8_OK;
}

template <int NKK, bool ROWS128>
int launch_bwd_dx_geometry(const BwdDxArgs& g, hipStream_t s) {
  const uint32_t ntile = g.tiles_m * g.tiles_k;
  const uint32_t want = ((ntile + 7u) / 8u) * 8u;
  const dim3 grid(want < 256u ? want : 256u), block(512);
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_dx_kernel<NKK, ROWS128>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kBwdLdsBytes) != hipSuccess)
    return MI355_W8A8_ERR_LAUNCH;
  hipLaunchKernelGGL((bwd_dx_kernel<NKK, ROWS128>), grid, block, kBwdLdsBytes, s, g);
  return launch_status();
}

template <int NKK>
int launch_bwd_dx(const BwdDxArgs& g, bool rows128, hipStream_t s) {
  return rows128 ? launch_bwd_dx_geometry<NKK, true>(g, s) : launch_bwd_dx_geometry<NKK, false>(g, s);
}

// The stages of a backward call behind its routing tables: dy into operand order (with the partial
// sums of r = dy @ B.T), r and z finished, the pull-back GEMM, the LoRA cotangents.  The dense call
// and the grouped call differ only in who wrote the tables and in the per-tile weights.
struct BwdBody {
  uint32_t m, k, n, n_groups, rank;
  const void* x; const void* dy; const void* w_packed;
  const void* lora_b; const float* lora_scaling;
  void* dx; void* d_lora_a; void* d_lora_b; float* d_lora_scaling;
  bool lora, want_grads, skip_prologue, skip_gemm;
  // tables (null: identity routing, everything in group 0)
  const int32_t* src_row; const int32_t* slot_group; const int32_t* blk_range; const int32_t* group_off;
  // grouped calls only
  const int32_t* skip_range;  // blk_range again when blocks without rows are to be skipped
  const int32_t* tile_weight; const int32_t* chunk_tab; const int32_t* chunk0; const int32_t* group_beg;
  const int32_t* group_end;
  size_t w_stride; uint32_t sw_stride;
  bool rows128;  // the pull-back runs 128-row x 512-k tiles (the tables are padded to match)
};

template <class Layout>
int launch_bwd_body(const BwdBody& b, const Layout& w, unsigned char* ws, hipStream_t s) {
  int st;
  if (!b.skip_prologue) {  // dy into operand order; the same pass leaves the partial sums of r = dy @ B.T
    BwdPackDyArgs d{};
    d.dy = static_cast<const uint16_t*>(b.dy);
    d.src_row = b.src_row; d.slot_group = b.slot_group; d.blk_range = b.blk_range;
    d.dyp = ws + w.dyp;
    d.lora_b = static_cast<const uint16_t*>(b.lora_b);
    d.rpart = b.lora ? reinterpret_cast<float*>(ws + w.rpart) : nullptr;
    d.M = b.m; d.N = b.n; d.NB = w.NB; d.n_row_blocks = w.slots / 32u; d.n_col_groups = w.N_pad / 128u;
    d.n_slices = w.n_slices; d.groups_per_slice = w.groups_per_slice; d.r = b.rank; d.slots = w.slots;
    const dim3 grid(d.n_row_blocks * d.n_slices), block(256);
    if (!b.lora) hipLaunchKernelGGL((bwd_pack_dy_kernel<0>), grid, block, 0, s, d);
    else if (w.nkk > 2u) hipLaunchKernelGGL((bwd_pack_dy_kernel<2>), grid, block, 0, s, d);
    else hipLaunchKernelGGL((bwd_pack_dy_kernel<1>), grid, block, 0, s, d);
    if ((st = launch_status())) return st;
  }
  if (b.lora && !b.skip_prologue) {
    {
      BwdRFinishArgs f{};
      f.rpart = reinterpret_cast<const float*>(ws + w.rpart);
      f.slot_group = b.slot_group;
      f.blk_range = b.skip_range;
      f.lora_scaling = b.lora_scaling;
      f.r_raw = reinterpret_cast<float*>(ws + w.r_raw);
      f.rs = reinterpret_cast<float*>(ws + w.rs);
      f.rp = ws + w.rp;
      f.n_slices = w.n_slices; f.slots = w.slots; f.nkk = w.nkk; f.cols = w.nkk > 2u ? 64u : 32u;
      hipLaunchKernelGGL(bwd_r_finish_kernel, dim3(w.slots / 32u), dim3(256), 0, s, f);
      if ((st = launch_status())) return st;
    }
    if (b.d_lora_b || b.d_lora_scaling) {  // z = x @ A, recomputed rather than saved by the forward
      LoraAArgs lz{};
      lz.xsrc = static_cast<const uint16_t*>(b.x);
      lz.at = reinterpret_cast<const uint16_t*>(ws + w.at);
      lz.src_row = b.src_row; lz.slot_group = b.slot_group; lz.blk_range = b.blk_range;
      lz.zp = nullptr;
      lz.M = b.m; lz.K = b.k; lz.r = b.rank; lz.nkk = w.nkk;
      lz.n_steps = (b.k + 63u) / 64u;
      lz.nterms = 3u;
      lz.n_blocks = w.slots / 32u;
      // K is cut into slices so that a call of few row blocks still fills the chip; the slices land
      // in the partial table (r's partials have been consumed, it holds n_slices of them) and are
      // added in slice order.  A slice keeps at least one 64-wide step for each of the 16 waves, and
      // the count depends on K and N only, so that a grouped call and the dense calls over its
      // groups add in the same order.
      const uint32_t by_steps = lz.n_steps / 16u ? lz.n_steps / 16u : 1u;
      const uint32_t nks = by_steps < w.n_slices ? by_steps : w.n_slices;
      lz.n_ksplit = nks;
      lz.steps_per_wave = ((lz.n_steps + nks - 1u) / nks + 15u) / 16u;
      lz.zf = reinterpret_cast<float*>(ws + w.rpart);
      lz.zf_stride = kBwdRankStride;
      lz.zf_slice = w.slots * kBwdRankStride;
      const dim3 grid(lz.n_blocks * nks), block(1024);
      (void)block;
      if ((st = launch_lora_a(lz, w.nkk, grid, s))) return st;
      BwdRFinishArgs f{};
      f.rpart = reinterpret_cast<const float*>(ws + w.rpart);
      f.blk_range = b.skip_range;
      f.r_raw = reinterpret_cast<float*>(ws + w.z);
      f.n_slices = nks; f.slots = w.slots; f.nkk = w.nkk; f.cols = w.nkk > 2u ? 64u : 32u;
      hipLaunchKernelGGL(bwd_r_finish_kernel, dim3(w.slots / 32u), dim3(256), 0, s, f);
      if ((st = launch_status())) return st;
    }
  }
  if (!b.skip_gemm) {
    BwdDxArgs g{};
    g.dyp = ws + w.dyp;
    g.wp = static_cast<const unsigned char*>(b.w_packed);
    g.swp = reinterpret_cast<const float*>(ws + w.swp);
    g.rp = b.lora ? ws + w.rp : nullptr;
    g.ap = b.lora ? ws + w.ap : nullptr;
    g.src_row = b.src_row; g.slot_group = b.slot_group; g.blk_range = b.blk_range;
    g.dx = static_cast<uint16_t*>(b.dx);
    g.M = b.m; g.K = b.k; g.KB = w.KB; g.NB = w.NB; g.tiles_m = w.tiles_m; g.tiles_k = w.tiles_k;
    g.tile_weight = b.tile_weight; g.w_stride = b.w_stride; g.sw_stride = b.sw_stride;
    switch (b.lora ? w.nkk : 0u) {
      case 0: st = launch_bwd_dx<0>(g, b.rows128, s); break;
      case 1: st = launch_bwd_dx<1>(g, b.rows128, s); break;
      case 2: st = launch_bwd_dx<2>(g, b.rows128, s); break;
      default: st = launch_bwd_dx<4>(g, b.rows128, s); break;
    }
    if (st) return st;
  }
  if (b.lora && b.want_grads) {
    BwdDloraArgs d{};
    d.x = static_cast<const uint16_t*>(b.x);
    d.dy = static_cast<const uint16_t*>(b.dy);
    d.rs = reinterpret_cast<const float*>(ws + w.rs);
    d.z = reinterpret_cast<const float*>(ws + w.z);
    d.src_row = b.src_row;
    d.group_off = b.group_off;
    d.chunk_tab = b.chunk_tab;
    d.partA = reinterpret_cast<float*>(ws + w.partA);
    d.partB = reinterpret_cast<float*>(ws + w.partB);
    d.M = b.m; d.K = b.k; d.N = b.n; d.n_groups = b.n_groups; d.max_chunks = w.max_chunks;
    d.col_tiles_a = b.d_lora_a ? (b.k + 255u) / 256u : 0u;
    d.col_tiles_b = b.d_lora_b ? (b.n + 255u) / 256u : 0u;
    if (d.col_tiles_a + d.col_tiles_b) {
      const dim3 grid(w.max_chunks * (d.col_tiles_a + d.col_tiles_b)), block(256);
      const uint32_t lds_bytes = (kBwdStageRows / 32u) * (w.R / 32u) * 6u * kBlockBytes;
      if (w.R == 32u) {
        hipLaunchKernelGGL((bwd_dlora_kernel<1>), grid, block, lds_bytes, s, d);
      } else {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&bwd_dlora_kernel<2>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
          return MI355_W8A8_ERR_LAUNCH;
        hipLaunchKernelGGL((bwd_dlora_kernel<2>), grid, block, lds_bytes, s, d);
      }
      if ((st = launch_status())) return st;
    }
    BwdReduceArgs r{};
    r.partA = d.partA; r.partB = d.partB;
    r.r_raw = reinterpret_cast<const float*>(ws + w.r_raw);
    r.z = d.z;
    r.lora_scaling = b.lora_scaling;
    r.group_off = b.group_off;
    r.chunk0_tab = b.chunk0; r.group_beg = b.group_beg; r.group_end = b.group_end;
    r.d_a = static_cast<uint16_t*>(b.d_lora_a);
    r.d_b = static_cast<uint16_t*>(b.d_lora_b);
    r.d_s = b.d_lora_scaling;
    r.K = b.k; r.N = b.n; r.r = b.rank; r.R = w.R; r.n_groups = b.n_groups;
    r.blocks_a = b.d_lora_a ? (uint32_t)(((uint64_t)b.n_groups * b.rank * b.k + 255u) / 256u) : 0u;
    r.blocks_b = b.d_lora_b ? (uint32_t)(((uint64_t)b.n_groups * b.rank * b.n / 4u + 255u) / 256u) : 0u;
    const uint32_t s_blocks = b.d_lora_scaling ? b.n_groups : 0u;
    hipLaunchKernelGGL(bwd_dlora_reduce_kernel, dim3(r.blocks_a + r.blocks_b + s_blocks), dim3(256), 0, s, r);
    if ((st = launch_status())) return st;
  }
  return MI355_W8A8_OK;
}

int run_backward(const mi355_w8a8_bwd_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_bwd_problem)) return MI355_W8A8_ERR_STRUCT;
  int st = validate_bwd_dims(p->m, p->k, p->n, p->n_adapters, p->rank);
  if (st) return st;
  if (p->flags & ~(MI355_W8A8_FLAG_SKIP_PROLOGUE | MI355_W8A8_FLAG_SKIP_GEMM)) return MI355_W8A8_ERR_SHAPE;
  const bool skip_prologue = (p->flags & MI355_W8A8_FLAG_SKIP_PROLOGUE) != 0;  // measurement: the workspace holds a previous call's tables
  const bool skip_gemm = (p->flags & MI355_W8A8_FLAG_SKIP_GEMM) != 0;
  if (!p->dy || !p->w_packed || !p->w_scales || !p->dx) return MI355_W8A8_ERR_NULL;
  const bool lora = p->n_adapters > 0;
  const bool want_grads = p->d_lora_a || p->d_lora_b || p->d_lora_scaling;
  if (lora) {
    if (!p->lora_a || !p->lora_b || !p->lora_scaling) return MI355_W8A8_ERR_NULL;
    if (want_grads && !p->x) return MI355_W8A8_ERR_NULL;
  } else if (p->adapter_indices || want_grads) {
    return MI355_W8A8_ERR_SHAPE;
  }
  if (!aligned16(p->x) || !aligned16(p->dy) || !aligned16(p->w_packed) || !aligned16(p->w_scales) ||
      !aligned16(p->lora_a) || !aligned16(p->lora_b) || !aligned16(p->dx) || !aligned16(p->d_lora_a) ||
      !aligned16(p->d_lora_b) || !aligned16(p->adapter_indices))
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t dx_bytes = (uint64_t)p->m * p->k * 2u, dy_bytes = (uint64_t)p->m * p->n * 2u;
  const uint64_t a_bytes = (uint64_t)p->n_adapters * p->rank * p->k * 2u, b_bytes = (uint64_t)p->n_adapters * p->rank * p->n * 2u;
  if (overlaps(p->dx, dx_bytes, p->dy, dy_bytes) || overlaps(p->dx, dx_bytes, p->x, dx_bytes) ||
      overlaps(p->dx, dx_bytes, p->workspace, p->workspace_bytes) ||
      overlaps(p->d_lora_a, a_bytes, p->lora_a, a_bytes) || overlaps(p->d_lora_b, b_bytes, p->lora_b, b_bytes) ||
      overlaps(p->d_lora_a, a_bytes, p->workspace, p->workspace_bytes) ||
      overlaps(p->d_lora_b, b_bytes, p->workspace, p->workspace_bytes) ||
      overlaps(p->d_lora_a, a_bytes, p->dx, dx_bytes) || overlaps(p->d_lora_b, b_bytes, p->dx, dx_bytes))
    return MI355_W8A8_ERR_ALIAS;
  const BwdLayout w = make_bwd_layout(p->m, p->k, p->n, p->n_adapters, lora ? p->rank : 0u);
  if (!p->workspace || p->workspace_bytes < w.total) return MI355_W8A8_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return MI355_W8A8_ERR_ALIGN;
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  const bool routed = lora && p->adapter_indices && p->n_adapters > 1;
  int32_t* src_row = reinterpret_cast<int32_t*>(ws + w.src_row);
  int32_t* slot_group = reinterpret_cast<int32_t*>(ws + w.slot_group);
  int32_t* blk_range = reinterpret_cast<int32_t*>(ws + w.blk_range);
  int32_t* group_off = reinterpret_cast<int32_t*>(ws + w.group_off);
  (void)hipGetLastError();

  if (!skip_prologue) {  // tables: routing, A transposed / in operand order, scales in packed column order
    BwdPrepArgs pa{};
    pa.idx = routed ? p->adapter_indices : nullptr;
    pa.src_row = src_row; pa.dst_pos = reinterpret_cast<int32_t*>(ws + w.dst_pos);
    pa.slot_group = slot_group; pa.blk_range = blk_range; pa.group_off = group_off;
    pa.lora_a = static_cast<const uint16_t*>(p->lora_a);
    pa.at = lora ? reinterpret_cast<uint16_t*>(ws + w.at) : nullptr;
    pa.ap = lora ? ws + w.ap : nullptr;
    pa.sw = p->w_scales; pa.swp = reinterpret_cast<float*>(ws + w.swp);
    pa.M = p->m; pa.K = p->k; pa.N = p->n; pa.N_pad = w.N_pad; pa.n_groups = p->n_adapters; pa.r = p->rank;
    pa.nkk = w.nkk; pa.kb32 = w.KB; pa.slots = w.slots;
    pa.route_blocks = lora ? 1u : 0u;
    pa.a_blocks = lora ? (uint32_t)(((uint64_t)p->n_adapters * p->k * ((p->rank + 7u) / 8u) + 1023u) / 1024u) : 0u;
    pa.ap_blocks = lora ? (uint32_t)(((uint64_t)p->n_adapters * w.KB * w.nkk * 64u + 1023u) / 1024u) : 0u;
    const uint32_t sw_blocks = (w.N_pad + 1023u) / 1024u;
    hipLaunchKernelGGL(bwd_prep_kernel, dim3(pa.route_blocks + pa.a_blocks + pa.ap_blocks + sw_blocks), dim3(1024), 0, s, pa);
    if ((st = launch_status())) return st;
  }
  BwdBody b{};
  b.m = p->m; b.k = p->k; b.n = p->n; b.n_groups = p->n_adapters; b.rank = p->rank;
  b.x = p->x; b.dy = p->dy; b.w_packed = p->w_packed; b.lora_b = p->lora_b; b.lora_scaling = p->lora_scaling;
  b.dx = p->dx; b.d_lora_a = p->d_lora_a; b.d_lora_b = p->d_lora_b; b.d_lora_scaling = p->d_lora_scaling;
  b.lora = lora; b.want_grads = want_grads; b.skip_prologue = skip_prologue; b.skip_gemm = skip_gemm;
  b.src_row = routed ? src_row : nullptr;
  b.slot_group = routed ? slot_group : nullptr;
  b.blk_range = routed ? blk_range : nullptr;
  b.group_off = group_off;
  return launch_bwd_body(b, w, ws, s);
}

// ---------------------------------------------------------------------------------------
// grouped (per-expert) backward
// ---------------------------------------------------------------------------------------
struct BwdGroupedLayout {
  uint64_t dyp, swp, src_row, dst_pos, slot_group, blk_range, group_beg, group_end, tile_weight, chunk_tab, chunk0,
      at, ap, rp, z, r_raw, rs, rpart, partA, partB, total;
  uint32_t slots, nkk, K_pad, KB, N_pad, NB, tiles_m, tiles_k, max_chunks, R, n_slices, groups_per_slice, n_weights,
      gpw, sw_stride, tile_rows;
};

BwdGroupedLayout make_bwd_grouped_layout(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank,
                                         uint32_t gpw_in) {
  BwdGroupedLayout w{};
  w.gpw = gpw_in ? gpw_in : 1u;
  w.n_weights = n_groups / w.gpw;
  w.K_pad = k_padded(k); w.KB = w.K_pad / 32u;
  w.N_pad = n_padded(n); w.NB = w.N_pad / 32u;
  // Tile geometry of the pull-back: 256 rows x 256 k, or 128 rows x 512 k (the same area).  The group sizes
  // live on the device, so the choice goes by the average rows per weight: a weight with r rows takes about
  // r / rows + 1/2 row tiles, and the geometry with fewer tiles in total wins (ties keep 256 rows).
  {
    const double avg = (double)m / (double)w.n_weights;
    const double t256 = (avg / 256.0 + 0.5) * (double)((w.KB + 7u) / 8u);
    const double t128 = (avg / 128.0 + 0.5) * (double)((w.KB + 15u) / 16u);
    w.tile_rows = t128 < t256 ? 128u : 256u;
  }
  // every weight with rows pads its slots to a multiple of the tile rows
  const uint32_t with_rows = w.n_weights < m ? w.n_weights : m;
  w.slots = round_up(m + (w.tile_rows - 1u) * with_rows, 256u);
  w.tiles_m = w.slots / w.tile_rows;
  w.tiles_k = w.tile_rows == 128u ? (w.KB + 15u) / 16u : (w.KB + 7u) / 8u;
  w.nkk = rank_chunks(rank);
  w.R = w.nkk > 2u ? 64u : 32u;
  w.max_chunks = (m + kBwdChunkRows - 1u) / kBwdChunkRows + n_groups;
  {
    const uint32_t ng = w.N_pad / 128u;
    w.n_slices = (ng + 3u) / 4u < 8u ? (ng + 3u) / 4u : 8u;
    w.groups_per_slice = (ng + w.n_slices - 1u) / w.n_slices;
  }
  w.sw_stride = w.N_pad + kBwdScalePad;
  uint64_t off = 0;
  w.dyp = off; off += align256((uint64_t)w.slots * w.N_pad * 2u);
  w.swp = off; off += align256((uint64_t)w.n_weights * w.sw_stride * 4u);
  w.src_row = off; off += align256((uint64_t)w.slots * 4u);
  w.dst_pos = off; off += align256((uint64_t)m * 4u);
  w.slot_group = off; off += align256((uint64_t)w.slots * 4u);
  w.blk_range = off; off += align256((uint64_t)(w.slots / 32u) * 4u);
  w.group_beg = off; off += align256((uint64_t)n_groups * 4u);
  w.group_end = off; off += align256((uint64_t)n_groups * 4u);
  w.tile_weight = off; off += align256((uint64_t)w.tiles_m * 4u);
  w.chunk_tab = off; off += align256((uint64_t)w.max_chunks * 12u);
  w.chunk0 = off; off += align256((uint64_t)(n_groups + 1u) * 4u);
  if (rank) {
    w.at = off; off += align256((uint64_t)n_groups * rank * k * 2u);
    w.ap = off; off += align256((uint64_t)n_groups * w.KB * w.nkk * kBlockBytes);
    w.rp = off; off += align256((uint64_t)(w.slots / 32u) * w.nkk * 3u * kBlockBytes);
    w.z = off; off += align256((uint64_t)w.slots * kBwdRankStride * 4u);
    w.r_raw = off; off += align256((uint64_t)w.slots * kBwdRankStride * 4u);
    w.rs = off; off += align256((uint64_t)w.slots * kBwdRankStride * 4u);
    w.rpart = off; off += align256((uint64_t)w.n_slices * w.slots * kBwdRankStride * 4u);
    w.partA = off; off += align256((uint64_t)w.max_chunks * w.R * k * 4u);
    w.partB = off; off += align256((uint64_t)w.max_chunks * w.R * n * 4u);
  }
  w.total = off;
  return w;
}

int validate_bwd_grouped_dims(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank, uint32_t gpw) {
  int st = validate_common(m, k, n);
  if (st) return st;
  if (n % 8u) return MI355_W8A8_ERR_UNSUPPORTED;
  if (n_groups == 0) return MI355_W8A8_ERR_SHAPE;
  if (gpw == 0) gpw = 1;
  if (n_groups % gpw) return MI355_W8A8_ERR_SHAPE;
  if (n_groups > (uint32_t)kMaxGroups || rank > (uint32_t)kMaxRank) return MI355_W8A8_ERR_UNSUPPORTED;
  // 32-bit element offsets into dx, and slots that stay below the row limit
  if ((uint64_t)m * k >= (1ull << 32) - (1ull << 20)) return MI355_W8A8_ERR_UNSUPPORTED;
  if ((uint64_t)m + 255ull * (n_groups / gpw) + 256ull > (uint64_t)kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  return MI355_W8A8_OK;
}

int run_grouped_backward(const mi355_w8a8_grouped_bwd_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_grouped_bwd_problem)) return MI355_W8A8_ERR_STRUCT;
  if (p->flags) return MI355_W8A8_ERR_SHAPE;
  int st = validate_bwd_grouped_dims(p->m, p->k, p->n, p->n_groups, p->rank, p->groups_per_weight);
  if (st) return st;
  if (!p->dy || !p->w_packed || !p->w_scales || !p->dx || !p->group_sizes) return MI355_W8A8_ERR_NULL;
  const bool lora = p->rank > 0;
  const bool want_grads = p->d_lora_a || p->d_lora_b || p->d_lora_scaling;
  if (lora) {
    if (!p->lora_a || !p->lora_b || !p->lora_scaling) return MI355_W8A8_ERR_NULL;
    if (want_grads && !p->x) return MI355_W8A8_ERR_NULL;
  } else if (p->lora_a || p->lora_b || want_grads) {
    return MI355_W8A8_ERR_SHAPE;
  }
  if (!aligned16(p->x) || !aligned16(p->dy) || !aligned16(p->w_packed) || !aligned16(p->w_scales) ||
      !aligned16(p->lora_a) || !aligned16(p->lora_b) || !aligned16(p->dx) || !aligned16(p->d_lora_a) ||
      !aligned16(p->d_lora_b) || (reinterpret_cast<uintptr_t>(p->group_sizes) & 3u))
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t dx_bytes = (uint64_t)p->m * p->k * 2u, dy_bytes = (uint64_t)p->m * p->n * 2u;
  const uint64_t a_bytes = (uint64_t)p->n_groups * p->rank * p->k * 2u, b_bytes = (uint64_t)p->n_groups * p->rank * p->n * 2u;
  if (overlaps(p->dx, dx_bytes, p->dy, dy_bytes) || overlaps(p->dx, dx_bytes, p->x, dx_bytes) ||
      overlaps(p->dx, dx_bytes, p->workspace, p->workspace_bytes) ||
      overlaps(p->d_lora_a, a_bytes, p->lora_a, a_bytes) || overlaps(p->d_lora_b, b_bytes, p->lora_b, b_bytes) ||
      overlaps(p->d_lora_a, a_bytes, p->workspace, p->workspace_bytes) ||
      overlaps(p->d_lora_b, b_bytes, p->workspace, p->workspace_bytes) ||
      overlaps(p->d_lora_a, a_bytes, p->dx, dx_bytes) || overlaps(p->d_lora_b, b_bytes, p->dx, dx_bytes))
    return MI355_W8A8_ERR_ALIAS;
  const BwdGroupedLayout w = make_bwd_grouped_layout(p->m, p->k, p->n, p->n_groups, p->rank, p->groups_per_weight);
  if (!p->workspace || p->workspace_bytes < w.total) return MI355_W8A8_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return MI355_W8A8_ERR_ALIGN;
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  BwdGroupTables tab{};
  tab.src_row = reinterpret_cast<int32_t*>(ws + w.src_row);
  tab.dst_pos = reinterpret_cast<int32_t*>(ws + w.dst_pos);
  tab.slot_group = reinterpret_cast<int32_t*>(ws + w.slot_group);
  tab.blk_range = reinterpret_cast<int32_t*>(ws + w.blk_range);
  tab.group_beg = reinterpret_cast<int32_t*>(ws + w.group_beg);
  tab.group_end = reinterpret_cast<int32_t*>(ws + w.group_end);
  tab.tile_weight = reinterpret_cast<int32_t*>(ws + w.tile_weight);
  tab.chunk_tab = reinterpret_cast<int32_t*>(ws + w.chunk_tab);
  tab.chunk0 = reinterpret_cast<int32_t*>(ws + w.chunk0);
  (void)hipGetLastError();

  {  // tables: routing, A transposed / in operand order, every weight's scales in packed column order
    BwdGroupedPrepArgs pa{};
    pa.group_sizes = p->group_sizes;
    pa.tab = tab;
    pa.lora_a = static_cast<const uint16_t*>(p->lora_a);
    pa.at = lora ? reinterpret_cast<uint16_t*>(ws + w.at) : nullptr;
    pa.ap = lora ? ws + w.ap : nullptr;
    pa.sw = p->w_scales; pa.swp = reinterpret_cast<float*>(ws + w.swp);
    pa.dx = static_cast<uint16_t*>(p->dx);
    pa.M = p->m; pa.K = p->k; pa.N = p->n; pa.N_pad = w.N_pad; pa.n_groups = p->n_groups; pa.gpw = w.gpw;
    pa.n_weights = w.n_weights; pa.r = p->rank; pa.nkk = w.nkk; pa.kb32 = w.KB; pa.slots = w.slots;
    pa.max_chunks = w.max_chunks; pa.sw_stride = w.sw_stride; pa.tile_rows = w.tile_rows;
    pa.a_blocks = lora ? (uint32_t)(((uint64_t)p->n_groups * p->k * ((p->rank + 7u) / 8u) + 1023u) / 1024u) : 0u;
    pa.ap_blocks = lora ? (uint32_t)(((uint64_t)p->n_groups * w.KB * w.nkk * 64u + 1023u) / 1024u) : 0u;
    pa.sw_blocks_per_weight = (w.N_pad + 1023u) / 1024u;
    hipLaunchKernelGGL(bwd_grouped_prep_kernel,
                       dim3(1u + pa.a_blocks + pa.ap_blocks + pa.sw_blocks_per_weight * w.n_weights), dim3(1024), 0, s, pa);
    if ((st = launch_status())) return st;
  }
  BwdBody b{};
  b.m = p->m; b.k = p->k; b.n = p->n; b.n_groups = p->n_groups; b.rank = p->rank;
  b.x = p->x; b.dy = p->dy; b.w_packed = p->w_packed; b.lora_b = p->lora_b; b.lora_scaling = p->lora_scaling;
  b.dx = p->dx; b.d_lora_a = p->d_lora_a; b.d_lora_b = p->d_lora_b; b.d_lora_scaling = p->d_lora_scaling;
  b.lora = lora; b.want_grads = want_grads;
  b.src_row = tab.src_row; b.slot_group = tab.slot_group; b.blk_range = tab.blk_range; b.skip_range = tab.blk_range;
  b.tile_weight = tab.tile_weight; b.chunk_tab = tab.chunk_tab; b.chunk0 = tab.chunk0;
  b.group_beg = tab.group_beg; b.group_end = tab.group_end;
  b.w_stride = (size_t)mi355_w8a8_packed_weight_bytes(p->k, p->n);
  b.sw_stride = w.sw_stride;
  b.rows128 = w.tile_rows == 128u;
  return launch_bwd_body(b, w, ws, s);
}

int run_qkv_post(const mi355_w8a8_qkv_post_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_qkv_post_problem)) return MI355_W8A8_ERR_STRUCT;
  if (p->flags) return MI355_W8A8_ERR_SHAPE;
  if (p->m == 0 || p->num_query_heads == 0 || p->num_kv_heads == 0 || p->head_dim == 0) return MI355_W8A8_ERR_SHAPE;
  if (p->num_query_heads % p->num_kv_heads) return MI355_W8A8_ERR_SHAPE;
  if ((p->head_dim & 1u) || (p->rotary_dim & 1u) || p->rotary_dim > p->head_dim) return MI355_W8A8_ERR_SHAPE;
  if (!(p->rope_theta > 0.0f) || !(p->rms_eps > 0.0f)) return MI355_W8A8_ERR_SHAPE;
  if (p->head_dim > kQkvMaxHeadDim || p->m > kMaxRows || p->num_query_heads > 1024u) return MI355_W8A8_ERR_UNSUPPORTED;
  const uint64_t width = ((uint64_t)p->num_query_heads * 2u + 2u * p->num_kv_heads) * p->head_dim;
  if (width * p->m >= (1ull << 32)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!p->fused || !p->q_norm_weight || !p->k_norm_weight || !p->positions || !p->q || !p->k || !p->v || !p->gate)
    return MI355_W8A8_ERR_NULL;
  if (!aligned16(p->fused) || !aligned16(p->q) || !aligned16(p->k) || !aligned16(p->v) || !aligned16(p->gate) ||
      !aligned16(p->q_norm_weight) || !aligned16(p->k_norm_weight) || (reinterpret_cast<uintptr_t>(p->positions) & 3u))
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t fused_bytes = width * p->m * 2u;
  const uint64_t q_bytes = (uint64_t)p->m * p->num_query_heads * p->head_dim * 2u;
  const uint64_t kv_bytes = (uint64_t)p->m * p->num_kv_heads * p->head_dim * 2u;
  if (overlaps(p->fused, fused_bytes, p->q, q_bytes) || overlaps(p->fused, fused_bytes, p->gate, q_bytes) ||
      overlaps(p->fused, fused_bytes, p->k, kv_bytes) || overlaps(p->fused, fused_bytes, p->v, kv_bytes) ||
      overlaps(p->q, q_bytes, p->gate, q_bytes) || overlaps(p->k, kv_bytes, p->v, kv_bytes) ||
      overlaps(p->q, q_bytes, p->k, kv_bytes) || overlaps(p->q, q_bytes, p->v, kv_bytes) ||
      overlaps(p->gate, q_bytes, p->k, kv_bytes) || overlaps(p->gate, q_bytes, p->v, kv_bytes))
    return MI355_W8A8_ERR_ALIAS;
  QkvPostArgs a{};
  a.fused = static_cast<const uint16_t*>(p->fused);
  a.q_w = p->q_norm_weight; a.k_w = p->k_norm_weight; a.pos = p->positions;
  a.q = static_cast<uint16_t*>(p->q); a.k = static_cast<uint16_t*>(p->k);
  a.v = static_cast<uint16_t*>(p->v); a.gate = static_cast<uint16_t*>(p->gate);
  a.M = p->m; a.Hq = p->num_query_heads; a.Hkv = p->num_kv_heads; a.D = p->head_dim; a.rot = p->rotary_dim;
  a.width = (uint32_t)width; a.theta = p->rope_theta; a.eps = p->rms_eps;
  (void)hipGetLastError();
  hipLaunchKernelGGL(qkv_post_kernel, dim3(p->m), dim3(256), 0, s, a);
  return launch_status();
}

// Workgroups of the QKV pull-back when the head-norm weights get cotangents: each leaves one partial.
inline uint32_t qkv_bwd_parts(uint32_t m) { return m < 1024u ? m : 1024u; }
inline uint64_t qkv_bwd_workspace_bytes(uint32_t m, uint32_t head_dim) {
  return (uint64_t)qkv_bwd_parts(m) * 2u * head_dim * 4u;
}

int run_qkv_post_bwd(const mi355_w8a8_qkv_post_bwd_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_qkv_post_bwd_problem)) return MI355_W8A8_ERR_STRUCT;
  if (p->flags) return MI355_W8A8_ERR_SHAPE;
  if (p->m == 0 || p->num_query_heads == 0 || p->num_kv_heads == 0 || p->head_dim == 0) return MI355_W8A8_ERR_SHAPE;
  if (p->num_query_heads % p->num_kv_heads) return MI355_W8A8_ERR_SHAPE;
  if ((p->head_dim & 1u) || (p->rotary_dim & 1u) || p->rotary_dim > p->head_dim) return MI355_W8A8_ERR_SHAPE;
  if (!(p->rope_theta > 0.0f) || !(p->rms_eps > 0.0f)) return MI355_W8A8_ERR_SHAPE;
  if (p->head_dim > kQkvMaxHeadDim || p->m > kMaxRows || p->num_query_heads > 1024u) return MI355_W8A8_ERR_UNSUPPORTED;
  const uint64_t width = ((uint64_t)p->num_query_heads * 2u + 2u * p->num_kv_heads) * p->head_dim;
  if (width * p->m >= (1ull << 32)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!p->fused || !p->q_norm_weight || !p->k_norm_weight || !p->positions || !p->d_q || !p->d_k || !p->d_v ||
      !p->d_gate || !p->d_fused)
    return MI355_W8A8_ERR_NULL;
  const bool wgrad = p->d_q_norm_weight != nullptr;
  if (wgrad != (p->d_k_norm_weight != nullptr)) return MI355_W8A8_ERR_NULL;
  if (!aligned16(p->fused) || !aligned16(p->d_q) || !aligned16(p->d_k) || !aligned16(p->d_v) || !aligned16(p->d_gate) ||
      !aligned16(p->d_fused) || !aligned16(p->q_norm_weight) || !aligned16(p->k_norm_weight) ||
      (reinterpret_cast<uintptr_t>(p->positions) & 3u))
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t fused_bytes = width * p->m * 2u;
  const uint64_t q_bytes = (uint64_t)p->m * p->num_query_heads * p->head_dim * 2u;
  const uint64_t kv_bytes = (uint64_t)p->m * p->num_kv_heads * p->head_dim * 2u;
  if (overlaps(p->d_fused, fused_bytes, p->fused, fused_bytes) || overlaps(p->d_fused, fused_bytes, p->d_q, q_bytes) ||
      overlaps(p->d_fused, fused_bytes, p->d_gate, q_bytes) || overlaps(p->d_fused, fused_bytes, p->d_k, kv_bytes) ||
      overlaps(p->d_fused, fused_bytes, p->d_v, kv_bytes))
    return MI355_W8A8_ERR_ALIAS;
  const uint32_t parts = qkv_bwd_parts(p->m);
  if (wgrad) {
    const uint64_t need = qkv_bwd_workspace_bytes(p->m, p->head_dim);
    if (!p->workspace) return MI355_W8A8_ERR_NULL;
    if (p->workspace_bytes < need) return MI355_W8A8_ERR_WORKSPACE;
    if (!aligned16(p->workspace) || (reinterpret_cast<uintptr_t>(p->d_q_norm_weight) & 3u) ||
        (reinterpret_cast<uintptr_t>(p->d_k_norm_weight) & 3u))
      return MI355_W8A8_ERR_ALIGN;
    if (overlaps(p->workspace, need, p->d_fused, fused_bytes) || overlaps(p->workspace, need, p->fused, fused_bytes) ||
        overlaps(p->d_q_norm_weight, p->head_dim * 4ull, p->d_k_norm_weight, p->head_dim * 4ull))
      return MI355_W8A8_ERR_ALIAS;
  }
  QkvPostBwdArgs a{};
  a.fused = static_cast<const uint16_t*>(p->fused);
  a.q_w = p->q_norm_weight; a.k_w = p->k_norm_weight; a.pos = p->positions;
  a.dq = static_cast<const uint16_t*>(p->d_q); a.dk = static_cast<const uint16_t*>(p->d_k);
  a.dv = static_cast<const uint16_t*>(p->d_v); a.dgate = static_cast<const uint16_t*>(p->d_gate);
  a.dfused = static_cast<uint16_t*>(p->d_fused);
  a.partial = wgrad ? static_cast<float*>(p->workspace) : nullptr;
  a.M = p->m; a.Hq = p->num_query_heads; a.Hkv = p->num_kv_heads; a.D = p->head_dim; a.rot = p->rotary_dim;
  a.width = (uint32_t)width; a.theta = p->rope_theta; a.eps = p->rms_eps;
  const bool vec4 = (p->head_dim & 3u) == 0;
  (void)hipGetLastError();
  if (wgrad) {
    if (vec4) hipLaunchKernelGGL((qkv_post_bwd_kernel<4, true>), dim3(parts), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((qkv_post_bwd_kernel<1, true>), dim3(parts), dim3(256), 0, s, a);
    int st;
    if ((st = launch_status())) return st;
    ColumnSumArgs c{};
    c.partial = a.partial; c.n_parts = parts; c.stride = 2u * p->head_dim; c.cols = p->head_dim;
    c.out = p->d_q_norm_weight; c.col0 = 0;
    hipLaunchKernelGGL(column_sum_kernel, dim3((p->head_dim + 15u) / 16u), dim3(256), 0, s, c);
    c.out = p->d_k_norm_weight; c.col0 = p->head_dim;
    hipLaunchKernelGGL(column_sum_kernel, dim3((p->head_dim + 15u) / 16u), dim3(256), 0, s, c);
  } else {
    if (vec4) hipLaunchKernelGGL((qkv_post_bwd_kernel<4, false>), dim3(p->m), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((qkv_post_bwd_kernel<1, false>), dim3(p->m), dim3(256), 0, s, a);
  }
  return launch_status();
}

// Row slices of the decoder-norm weight cotangent: each leaves one partial row.
inline uint32_t rms_dgamma_slices(uint32_t m) { return m < 256u ? m : 256u; }
inline uint64_t delta_rms_bwd_workspace_bytes(uint32_t m, uint32_t k) {
  return (uint64_t)round_up(m, 64u) * 4u + (uint64_t)rms_dgamma_slices(m) * k * 4u;
}

int run_delta_rms_norm_bwd(const void* x, const float* gamma, const void* d_normalized, void* d_x, float* d_gamma,
                           void* workspace, uint64_t workspace_bytes, uint32_t m, uint32_t k, float eps,
                           hipStream_t s) {
  if (!x || !gamma || !d_normalized || !d_x) return MI355_W8A8_ERR_NULL;
  if (m == 0 || k == 0 || !(eps > 0.0f)) return MI355_W8A8_ERR_SHAPE;
  if (m > kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(d_normalized) || !aligned16(d_x) || !aligned16(gamma)) return MI355_W8A8_ERR_ALIGN;
  const uint64_t bytes = (uint64_t)m * k * 2u;
  if (overlaps(d_x, bytes, x, bytes) || overlaps(d_x, bytes, gamma, (uint64_t)k * 4u)) return MI355_W8A8_ERR_ALIAS;
  const uint64_t need = delta_rms_bwd_workspace_bytes(m, k);
  if (d_gamma) {
    // the weight cotangent reads d_normalized after the row pull-back has written d_x
    if (overlaps(d_x, bytes, d_normalized, bytes)) return MI355_W8A8_ERR_ALIAS;
    if (!workspace) return MI355_W8A8_ERR_NULL;
    if (workspace_bytes < need) return MI355_W8A8_ERR_WORKSPACE;
    if (!aligned16(workspace) || (reinterpret_cast<uintptr_t>(d_gamma) & 3u)) return MI355_W8A8_ERR_ALIGN;
    if (overlaps(workspace, need, d_x, bytes) || overlaps(workspace, need, x, bytes) ||
        overlaps(workspace, need, d_normalized, bytes) || overlaps(d_gamma, (uint64_t)k * 4u, d_x, bytes))
      return MI355_W8A8_ERR_ALIAS;
  } else if (d_x != d_normalized && overlaps(d_x, bytes, d_normalized, bytes)) {
    return MI355_W8A8_ERR_ALIAS;
  }
  DeltaRmsBwdArgs a{};
  a.x = static_cast<const uint16_t*>(x);
  a.gamma = gamma;
  a.dn = static_cast<const uint16_t*>(d_normalized);
  a.dx = static_cast<uint16_t*>(d_x);
  a.inv_out = d_gamma ? static_cast<float*>(workspace) : nullptr;
  a.M = m; a.K = k; a.eps = eps;
  (void)hipGetLastError();
  if ((k & 7u) == 0) hipLaunchKernelGGL((delta_rms_norm_bwd_kernel<true>), dim3(m), dim3(256), 0, s, a);
  else hipLaunchKernelGGL((delta_rms_norm_bwd_kernel<false>), dim3(m), dim3(256), 0, s, a);
  int st;
  if ((st = launch_status())) return st;
  if (d_gamma) {
    const uint32_t slices = rms_dgamma_slices(m);
    RmsDgammaArgs g{};
    g.x = a.x; g.dn = a.dn; g.inv = a.inv_out;
    g.partial = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + (uint64_t)round_up(m, 64u) * 4u);
    g.M = m; g.K = k;
    hipLaunchKernelGGL(rms_dgamma_partial_kernel, dim3((k + 255u) / 256u, slices), dim3(256), 0, s, g);
    if ((st = launch_status())) return st;
    ColumnSumArgs c{};
    c.partial = g.partial; c.n_parts = slices; c.stride = k; c.cols = k; c.col0 = 0; c.out = d_gamma;
    hipLaunchKernelGGL(column_sum_kernel, dim3((k + 15u) / 16u), dim3(256), 0, s, c);
    return launch_status();
  }
  return MI355_W8A8_OK;
}

int run_swiglu_bwd(const void* fused, const void* d_product, void* d_fused, uint32_t m, uint32_t n, hipStream_t s) {
  if (!fused || !d_product || !d_fused) return MI355_W8A8_ERR_NULL;
  if (m == 0 || n == 0 || (n & 7u)) return MI355_W8A8_ERR_SHAPE;
  if (m > kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(fused) || !aligned16(d_fused) || (reinterpret_cast<uintptr_t>(d_product) & 7u))
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t fused_bytes = (uint64_t)m * n * 2u;
  // d_fused may be fused itself (element i is read and written by the same thread), nothing else
  if (d_fused != fused && overlaps(d_fused, fused_bytes, fused, fused_bytes)) return MI355_W8A8_ERR_ALIAS;
  if (overlaps(d_fused, fused_bytes, d_product, fused_bytes / 2u)) return MI355_W8A8_ERR_ALIAS;
  SwigluBwdArgs a{};
  a.fused = static_cast<const uint16_t*>(fused);
  a.dprod = static_cast<const uint16_t*>(d_product);
  a.dfused = static_cast<uint16_t*>(d_fused);
  a.n_chunks = (uint64_t)m * n / 8u;
  const uint64_t blocks = (a.n_chunks + 255u) / 256u;
  (void)hipGetLastError();
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3((uint32_t)(blocks < 16384u ? blocks : 16384u)), dim3(256), 0, s, a);
  return launch_status();
}

int run_swiglu_fwd(const void* fused, void* product, uint32_t m, uint32_t n, hipStream_t s) {
  if (!fused || !product) return MI355_W8A8_ERR_NULL;
  if (m == 0 || n == 0 || (n & 7u)) return MI355_W8A8_ERR_SHAPE;
  if (m > kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(fused) || (reinterpret_cast<uintptr_t>(product) & 7u)) return MI355_W8A8_ERR_ALIGN;
  if (overlaps(product, (uint64_t)m * n, fused, (uint64_t)m * n * 2u)) return MI355_W8A8_ERR_ALIAS;
  SwigluFwdArgs a{};
  a.fused = static_cast<const uint16_t*>(fused);
  a.product = static_cast<uint16_t*>(product);
  a.n_chunks = (uint64_t)m * n / 8u;
  const uint64_t blocks = (a.n_chunks + 255u) / 256u;
  (void)hipGetLastError();
  hipLaunchKernelGGL(swiglu_fwd_kernel, dim3((uint32_t)(blocks < 16384u ? blocks : 16384u)), dim3(256), 0, s, a);
  return launch_status();
}

int run_rms_norm_bwd(const void* x, const float* gamma, const void* d_normalized, void* d_x, uint32_t m, uint32_t k,
                     float eps, hipStream_t s) {
  if (!x || !gamma || !d_normalized || !d_x) return MI355_W8A8_ERR_NULL;
  if (m == 0 || k == 0 || !(eps > 0.0f)) return MI355_W8A8_ERR_SHAPE;
  if (m > kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(d_normalized) || !aligned16(d_x) || !aligned16(gamma)) return MI355_W8A8_ERR_ALIGN;
  const uint64_t bytes = (uint64_t)m * k * 2u;
  // d_x may be d_normalized itself (a row is reduced before any of it is rewritten, element i by
  // the thread that reads it), nothing else
  if (d_x != d_normalized && overlaps(d_x, bytes, d_normalized, bytes)) return MI355_W8A8_ERR_ALIAS;
  if (overlaps(d_x, bytes, x, bytes) || overlaps(d_x, bytes, gamma, (uint64_t)k * 4u)) return MI355_W8A8_ERR_ALIAS;
  RmsNormBwdArgs a{};
  a.x = static_cast<const uint16_t*>(x);
  a.gamma = gamma;
  a.dn = static_cast<const uint16_t*>(d_normalized);
  a.dx = static_cast<uint16_t*>(d_x);
  a.M = m; a.K = k; a.eps = eps;
  (void)hipGetLastError();
  if ((k & 7u) == 0) hipLaunchKernelGGL((rms_norm_bwd_kernel<true>), dim3(m), dim3(256), 0, s, a);
  else hipLaunchKernelGGL((rms_norm_bwd_kernel<false>), dim3(m), dim3(256), 0, s, a);
  return launch_status();
}


int run_moe_route(const float* logits, uint32_t t, uint32_t e, uint32_t top_k, uint32_t norm, float* weights,
                  int32_t* selected, hipStream_t s) {
  if (!logits || !weights || !selected) return MI355_W8A8_ERR_NULL;
  if (t == 0 || e == 0 || top_k == 0 || top_k > e || norm > 1u) return MI355_W8A8_ERR_SHAPE;
  if (e > kMoeMaxExperts || top_k > kMoeMaxTopK || t > kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(weights) |
       reinterpret_cast<uintptr_t>(selected)) & 3u)
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t out_bytes = (uint64_t)t * top_k * 4u;
  if (overlaps(weights, out_bytes, logits, (uint64_t)t * e * 4u) ||
      overlaps(selected, out_bytes, logits, (uint64_t)t * e * 4u) || overlaps(weights, out_bytes, selected, out_bytes))
    return MI355_W8A8_ERR_ALIAS;
  MoeRouteArgs a{};
  a.logits = logits; a.weights = weights; a.selected = selected;
  a.T = t; a.E = e; a.top_k = top_k; a.norm = norm;
  (void)hipGetLastError();
  const dim3 grid((t + 3u) / 4u), block(256);
  if (e <= 64u) hipLaunchKernelGGL((moe_route_kernel<1>), grid, block, 0, s, a);
  else if (e <= 128u) hipLaunchKernelGGL((moe_route_kernel<2>), grid, block, 0, s, a);
  else if (e <= 256u) hipLaunchKernelGGL((moe_route_kernel<4>), grid, block, 0, s, a);
  else if (e <= 512u) hipLaunchKernelGGL((moe_route_kernel<8>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((moe_route_kernel<16>), grid, block, 0, s, a);
  return launch_status();
}

int run_moe_route_bwd(const float* logits, const int32_t* selected, const float* d_weights, uint32_t t, uint32_t e,
                      uint32_t top_k, uint32_t norm, float* d_logits, hipStream_t s) {
  if (!logits || !selected || !d_weights || !d_logits) return MI355_W8A8_ERR_NULL;
  if (t == 0 || e == 0 || top_k == 0 || top_k > e || norm > 1u) return MI355_W8A8_ERR_SHAPE;
  if (e > kMoeMaxExperts || top_k > kMoeMaxTopK || t > kMaxRows) return MI355_W8A8_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(selected) |
       reinterpret_cast<uintptr_t>(d_weights) | reinterpret_cast<uintptr_t>(d_logits)) & 3u)
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t tab_bytes = (uint64_t)t * top_k * 4u, row_bytes = (uint64_t)t * e * 4u;
  // d_logits may be the logits buffer itself (a token's row is read whole before it is rewritten), nothing else
  if (d_logits != logits && overlaps(d_logits, row_bytes, logits, row_bytes)) return MI355_W8A8_ERR_ALIAS;
  if (overlaps(d_logits, row_bytes, selected, tab_bytes) || overlaps(d_logits, row_bytes, d_weights, tab_bytes))
    return MI355_W8A8_ERR_ALIAS;
  MoeRouteBwdArgs a{};
  a.logits = logits; a.selected = selected; a.d_weights = d_weights; a.d_logits = d_logits;
  a.T = t; a.E = e; a.top_k = top_k; a.norm = norm;
  (void)hipGetLastError();
  const dim3 grid((t + 3u) / 4u), block(256);
  if (e <= 64u) hipLaunchKernelGGL((moe_route_bwd_kernel<1>), grid, block, 0, s, a);
  else if (e <= 128u) hipLaunchKernelGGL((moe_route_bwd_kernel<2>), grid, block, 0, s, a);
  else if (e <= 256u) hipLaunchKernelGGL((moe_route_bwd_kernel<4>), grid, block, 0, s, a);
  else if (e <= 512u) hipLaunchKernelGGL((moe_route_bwd_kernel<8>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((moe_route_bwd_kernel<16>), grid, block, 0, s, a);
  return launch_status();
}

struct MoeSortLayout { uint64_t chunk_cnt, group_start, total; uint32_t n_chunks; };

MoeSortLayout make_moe_sort_layout(uint32_t n_pairs, uint32_t n_groups) {
  MoeSortLayout L{};
  L.n_chunks = (n_pairs + kMoeChunk - 1u) / kMoeChunk;
  L.chunk_cnt = 0;
  L.group_start = ((uint64_t)L.n_chunks * n_groups * 4u + 255u) & ~255ull;
  L.total = L.group_start + (((uint64_t)n_groups * 4u + 255u) & ~255ull);
  return L;
}

int validate_moe_sort_dims(uint32_t n_pairs, uint32_t n_groups) {
  if (n_pairs == 0 || n_groups == 0) return MI355_W8A8_ERR_SHAPE;
  if (n_groups > kMoeMaxExperts || n_pairs > (1u << 30)) return MI355_W8A8_ERR_UNSUPPORTED;
  return MI355_W8A8_OK;
}

int run_moe_dispatch(const mi355_w8a8_moe_dispatch_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_moe_dispatch_problem)) return MI355_W8A8_ERR_STRUCT;
  if (p->flags) return MI355_W8A8_ERR_SHAPE;
  int st = validate_moe_sort_dims(p->n_pairs, p->n_groups);
  if (st) return st;
  if (p->repeat == 0 || p->n_pairs % p->repeat) return MI355_W8A8_ERR_SHAPE;
  if (!p->indices || !p->group_sizes || !p->sort_indices || !p->unsort_indices) return MI355_W8A8_ERR_NULL;
  if ((p->adapter_indices != nullptr) != (p->sorted_adapters != nullptr)) return MI355_W8A8_ERR_NULL;
  if ((p->tokens != nullptr) != (p->sorted_tokens != nullptr)) return MI355_W8A8_ERR_NULL;
  if (p->tokens && (p->width == 0 || (p->width & 7u))) return MI355_W8A8_ERR_SHAPE;
  if (!aligned16(p->tokens) || !aligned16(p->sorted_tokens)) return MI355_W8A8_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(p->indices) | reinterpret_cast<uintptr_t>(p->group_sizes) |
       reinterpret_cast<uintptr_t>(p->sort_indices) | reinterpret_cast<uintptr_t>(p->unsort_indices) |
       reinterpret_cast<uintptr_t>(p->adapter_indices) | reinterpret_cast<uintptr_t>(p->sorted_adapters)) & 3u)
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t idx_bytes = (uint64_t)p->n_pairs * 4u;
  if (p->tokens) {
    const uint64_t out_bytes = (uint64_t)p->n_pairs * p->width * 2u;
    if (overlaps(p->sorted_tokens, out_bytes, p->tokens, out_bytes / p->repeat) ||
        overlaps(p->sorted_tokens, out_bytes, p->indices, idx_bytes) ||
        overlaps(p->sorted_tokens, out_bytes, p->sort_indices, idx_bytes) ||
        overlaps(p->sorted_tokens, out_bytes, p->unsort_indices, idx_bytes))
      return MI355_W8A8_ERR_ALIAS;
  }
  if (overlaps(p->sort_indices, idx_bytes, p->indices, idx_bytes) ||
      overlaps(p->unsort_indices, idx_bytes, p->indices, idx_bytes) ||
      overlaps(p->sort_indices, idx_bytes, p->unsort_indices, idx_bytes))
    return MI355_W8A8_ERR_ALIAS;
  const MoeSortLayout L = make_moe_sort_layout(p->n_pairs, p->n_groups);
  if (!p->workspace || p->workspace_bytes < L.total) return MI355_W8A8_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return MI355_W8A8_ERR_ALIGN;
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  MoeSortArgs a{};
  a.indices = p->indices;
  a.tokens = static_cast<const uint16_t*>(p->tokens);
  a.adapters = p->adapter_indices;
  a.sorted_tokens = static_cast<uint16_t*>(p->sorted_tokens);
  a.group_sizes = p->group_sizes;
  a.sort_indices = p->sort_indices;
  a.unsort_indices = p->unsort_indices;
  a.sorted_adapters = p->sorted_adapters;
  a.chunk_cnt = reinterpret_cast<int32_t*>(ws + L.chunk_cnt);
  a.group_start = reinterpret_cast<int32_t*>(ws + L.group_start);
  a.P = p->n_pairs; a.G = p->n_groups; a.repeat = p->repeat; a.width = p->width; a.n_chunks = L.n_chunks;
  (void)hipGetLastError();
  hipLaunchKernelGGL(moe_hist_kernel, dim3(L.n_chunks), dim3(1024), 0, s, a);
  if ((st = launch_status())) return st;
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(1024), 0, s, a);
  if ((st = launch_status())) return st;
  hipLaunchKernelGGL(moe_scatter_kernel, dim3(L.n_chunks), dim3(1024), 0, s, a);
  if ((st = launch_status()) || !a.tokens) return st;
  if (p->repeat > 1u)
    hipLaunchKernelGGL(moe_spread_kernel, dim3((p->n_pairs / p->repeat + 3u) / 4u), dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL(moe_gather_kernel, dim3((p->n_pairs + 7u) / 8u), dim3(256), 0, s, a);
  return launch_status();
}

int run_moe_combine(const void* expert_out, const int32_t* unsort, const float* weights, void* out, uint32_t t,
                    uint32_t top_k, uint32_t width, hipStream_t s) {
  if (!expert_out || !unsort || !weights || !out) return MI355_W8A8_ERR_NULL;
  if (t == 0 || top_k == 0 || width == 0 || (width & 7u)) return MI355_W8A8_ERR_SHAPE;
  if (top_k > kMoeMaxTopK || t > kMaxRows || (uint64_t)t * top_k > (1ull << 30)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(expert_out) || !aligned16(out)) return MI355_W8A8_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(unsort) | reinterpret_cast<uintptr_t>(weights)) & 3u) return MI355_W8A8_ERR_ALIGN;
  const uint64_t out_bytes = (uint64_t)t * width * 2u;
  if (overlaps(out, out_bytes, expert_out, out_bytes * top_k) || overlaps(out, out_bytes, unsort, (uint64_t)t * top_k * 4u) ||
      overlaps(out, out_bytes, weights, (uint64_t)t * top_k * 4u))
    return MI355_W8A8_ERR_ALIAS;
  MoeCombineArgs a{};
  a.expert_out = static_cast<const uint16_t*>(expert_out);
  a.unsort = unsort; a.weights = weights;
  a.out = static_cast<uint16_t*>(out);
  a.T = t; a.top_k = top_k; a.width = width;
  (void)hipGetLastError();
  hipLaunchKernelGGL(moe_combine_kernel, dim3(t), dim3(256), 0, s, a);
  return launch_status();
}

int run_moe_combine_bwd(const void* d_out, const void* expert_out, const int32_t* sort, const float* weights,
                        void* d_expert_out, float* d_weights, uint32_t t, uint32_t top_k, uint32_t width, hipStream_t s) {
  if (!d_out || !sort || !weights || !d_expert_out) return MI355_W8A8_ERR_NULL;
  if (d_weights && !expert_out) return MI355_W8A8_ERR_NULL;
  if (t == 0 || top_k == 0 || width == 0 || (width & 7u)) return MI355_W8A8_ERR_SHAPE;
  if (top_k > kMoeMaxTopK || t > kMaxRows || (uint64_t)t * top_k > (1ull << 30)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(d_out) || !aligned16(expert_out) || !aligned16(d_expert_out)) return MI355_W8A8_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(sort) | reinterpret_cast<uintptr_t>(weights) | reinterpret_cast<uintptr_t>(d_weights)) & 3u)
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t tok_bytes = (uint64_t)t * width * 2u, pair_bytes = tok_bytes * top_k, tab_bytes = (uint64_t)t * top_k * 4u;
  if (overlaps(d_expert_out, pair_bytes, d_out, tok_bytes) || overlaps(d_expert_out, pair_bytes, expert_out, pair_bytes) ||
      overlaps(d_expert_out, pair_bytes, sort, tab_bytes) || overlaps(d_expert_out, pair_bytes, weights, tab_bytes) ||
      overlaps(d_weights, tab_bytes, weights, tab_bytes) || overlaps(d_weights, tab_bytes, d_expert_out, pair_bytes) ||
      overlaps(d_weights, tab_bytes, sort, tab_bytes))
    return MI355_W8A8_ERR_ALIAS;
  MoeCombineBwdArgs a{};
  a.d_out = static_cast<const uint16_t*>(d_out);
  a.expert_out = d_weights ? static_cast<const uint16_t*>(expert_out) : nullptr;
  a.sort = sort; a.weights = weights;
  a.d_expert_out = static_cast<uint16_t*>(d_expert_out);
  a.d_weights = d_weights;
  a.P = t * top_k; a.top_k = top_k; a.width = width;
  (void)hipGetLastError();
  hipLaunchKernelGGL(moe_combine_bwd_kernel, dim3((a.P + 7u) / 8u), dim3(256), 0, s, a);
  return launch_status();
}

constexpr uint32_t kGqZSlices = 32;
// K slices of the routed LoRA-A projection: one workgroup per 32-row block and slice, so that calls with
// fewer row blocks than the chip has CUs still fill it (the consumer adds the slices in order)
inline uint32_t gq_z_ksplit(uint32_t m_pad, uint32_t k) {
  const uint32_t n_blocks = m_pad / 32u, n_steps = (k + 63u) / 64u;
  uint32_t ks = n_blocks >= 192u ? 1u : (256u + n_blocks - 1u) / n_blocks;
  if (ks > 4u) ks = 4u;
  while (ks > 1u && n_steps / ks < 16u) --ks;  // every wave of a slice keeps at least one step
  return ks;
}
struct GqLayout { uint64_t codes, scales, z, src_row, dst_pos, slot_group, blk_range, at, total; uint32_t m_pad, G; };

GqLayout make_gq_layout(uint32_t m, uint32_t k_pad, uint32_t group, uint32_t n_adapters, uint32_t rank) {
  GqLayout L{};
  L.m_pad = round_up(m, 32u);
  L.G = k_pad / group;
  uint64_t off = 0;
  L.codes = off; off += align256((uint64_t)L.m_pad * k_pad);
  L.scales = off; off += align256((uint64_t)L.m_pad * L.G * 4u);
  // decode (one row block): LoRA-A arrives as up to kGqZSlices slices over K
  L.z = off; off += rank ? align256((uint64_t)L.m_pad * 64u * 4u * (L.m_pad == 32u ? kGqZSlices : 4u)) : 0u;
  L.src_row = off; off += rank ? align256((uint64_t)L.m_pad * 4u) : 0u;
  L.dst_pos = off; off += rank ? align256((uint64_t)L.m_pad * 4u) : 0u;
  L.slot_group = off; off += rank ? align256((uint64_t)L.m_pad * 4u) : 0u;
  L.blk_range = off; off += rank ? align256((uint64_t)(L.m_pad / 32u) * 4u) : 0u;
  // LoRA A in lora_a_kernel's operand order: per adapter and 64-wide k step 4 KiB per 32 rank columns
  L.at = off; off += (rank && n_adapters <= (uint32_t)kMaxAdapters)
                         ? align256((uint64_t)n_adapters * ((k_pad + 63u) / 64u) * (rank_chunks(rank) > 2u ? 2u : 1u) * 4u * kBlockBytes)
                         : 0u;
  L.total = off;
  return L;
}

int validate_gq_dims(uint32_t m, uint32_t k_pad, uint32_t group, uint32_t rank) {
  if (m == 0 || k_pad == 0 || group == 0) return MI355_W8A8_ERR_SHAPE;
  if ((group & 31u) || k_pad % group) return MI355_W8A8_ERR_UNSUPPORTED;
  if (m > kMaxRows || k_pad > kMaxK || rank > (uint32_t)kMaxRank) return MI355_W8A8_ERR_UNSUPPORTED;
  return MI355_W8A8_OK;
}

int run_gq_pack(const void* codes, void* packed, uint32_t k_pad, uint32_t n, uint32_t bits, hipStream_t s) {
  if (!codes || !packed) return MI355_W8A8_ERR_NULL;
  if (k_pad == 0 || n == 0 || (bits != 4u && bits != 8u)) return MI355_W8A8_ERR_SHAPE;
  if ((k_pad & 31u) || k_pad > kMaxK || n > kMaxN) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(packed)) return MI355_W8A8_ERR_ALIGN;
  const uint64_t src_bytes = (uint64_t)k_pad * n / (bits == 4u ? 2u : 1u);
  if (overlaps(packed, gq_packed_bytes(k_pad, n, bits), codes, src_bytes)) return MI355_W8A8_ERR_ALIAS;
  GqPackArgs a{};
  a.codes = static_cast<const unsigned char*>(codes);
  a.packed = static_cast<unsigned char*>(packed);
  a.k_pad = k_pad; a.n = n; a.bits = bits;
  a.n_items = (uint64_t)((n + 31u) / 32u) * (k_pad / 32u) * 64u;
  (void)hipGetLastError();
  hipLaunchKernelGGL(gq_pack_weight_kernel, dim3((uint32_t)((a.n_items + 255u) / 256u)), dim3(256), 0, s, a);
  return launch_status();
}

int run_gq_linear(const mi355_w8a8_gq_problem* p, hipStream_t s) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_gq_problem)) return MI355_W8A8_ERR_STRUCT;
  if (p->flags & ~MI355_W8A8_FLAG_GQ_DIRECT) return MI355_W8A8_ERR_SHAPE;
  int st = validate_gq_dims(p->m, p->k_pad, p->group_size, p->rank);
  if (st) return st;
  if (p->n == 0 || p->k == 0 || p->k > p->k_pad) return MI355_W8A8_ERR_SHAPE;
  if ((p->weight_bits != 4u && p->weight_bits != 8u) || (p->activation_bits != 4u && p->activation_bits != 8u))
    return MI355_W8A8_ERR_SHAPE;
  if (p->n > kMaxN || (uint64_t)p->m * p->n >= (1ull << 32)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!p->x || !p->w_packed || !p->w_scales || !p->out) return MI355_W8A8_ERR_NULL;
  const bool lora = p->n_adapters > 0;
  if (lora) {
    if (!p->lora_a || !p->lora_b || !p->lora_scaling) return MI355_W8A8_ERR_NULL;
    if (p->rank == 0 || p->n_adapters > (uint32_t)kMaxGroups) return MI355_W8A8_ERR_UNSUPPORTED;
  } else if (p->adapter_indices) {
    return MI355_W8A8_ERR_SHAPE;
  }
  if (!aligned16(p->w_packed) || (reinterpret_cast<uintptr_t>(p->x) & 1u) || (reinterpret_cast<uintptr_t>(p->out) & 1u) ||
      (reinterpret_cast<uintptr_t>(p->w_scales) & 3u) || (reinterpret_cast<uintptr_t>(p->adapter_indices) & 3u))
    return MI355_W8A8_ERR_ALIGN;
  const uint64_t out_bytes = (uint64_t)p->m * p->n * 2u;
  if (overlaps(p->out, out_bytes, p->x, (uint64_t)p->m * p->k * 2u) ||
      overlaps(p->out, out_bytes, p->w_packed, gq_packed_bytes(p->k_pad, p->n, p->weight_bits)) ||
      overlaps(p->out, out_bytes, p->workspace, p->workspace_bytes))
    return MI355_W8A8_ERR_ALIAS;
  const GqLayout L = make_gq_layout(p->m, p->k_pad, p->group_size, p->n_adapters, lora ? p->rank : 0u);
  if (!p->workspace || p->workspace_bytes < L.total) return MI355_W8A8_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return MI355_W8A8_ERR_ALIGN;
  unsigned char* ws = static_cast<unsigned char*>(p->workspace);
  (void)hipGetLastError();

  GqQuantArgs q{};
  q.x = static_cast<const uint16_t*>(p->x);
  q.codes = reinterpret_cast<int8_t*>(ws + L.codes);
  q.scales = reinterpret_cast<float*>(ws + L.scales);
  q.codes_rm = p->aux_x_codes; q.scales_rm = p->aux_x_scales;
  q.M = p->m; q.M_pad = L.m_pad; q.K = p->k; q.K_pad = p->k_pad; q.group = p->group_size; q.G = L.G;
  q.qmax = p->activation_bits == 4u ? 7.0f : 127.0f;
  // few rows: a row's groups are dealt to several waves so that the launch still fills the chip
  const uint32_t q_slices = L.m_pad >= 1024u ? 1u : (L.G < 16u ? L.G : 16u);
  q.groups_per_slice = (L.G + q_slices - 1u) / q_slices;
  hipLaunchKernelGGL(gq_quant_kernel, dim3(L.m_pad / 4u, (L.G + q.groups_per_slice - 1u) / q.groups_per_slice), dim3(256),
                     0, s, q);
  if ((st = launch_status())) return st;

  // z = x @ A[idx]: rows routed by adapter and multiplied on the matrix core (the kernels of the
  // per-channel path) when the adapter count and K allow it, else one wave per row
  const bool decode = L.m_pad == 32u;  // few rows: a wave per (row, k slice) instead of one row block
  const bool fast_z = lora && !decode && p->n_adapters <= (uint32_t)kMaxAdapters && (p->k & 7u) == 0 &&
                      aligned16(p->x) && aligned16(p->lora_a);
  const bool routed = fast_z && p->adapter_indices && p->n_adapters > 1u;
  int32_t* dst_pos = reinterpret_cast<int32_t*>(ws + L.dst_pos);
  uint32_t z_slices = 1u, z_slice_stride = p->m * 64u;
  if (fast_z) {
    int32_t* src_row = reinterpret_cast<int32_t*>(ws + L.src_row);
    int32_t* slot_group = reinterpret_cast<int32_t*>(ws + L.slot_group);
    int32_t* blk_range = reinterpret_cast<int32_t*>(ws + L.blk_range);
    uint16_t* at = reinterpret_cast<uint16_t*>(ws + L.at);
    LoraPrepArgs pa{};
    pa.idx = routed ? p->adapter_indices : nullptr;
    pa.src_row = src_row; pa.dst_pos = dst_pos; pa.slot_group = slot_group; pa.blk_range = blk_range;
    pa.lora_a = static_cast<const uint16_t*>(p->lora_a);
    pa.at = at;
    pa.M = p->m; pa.K = p->k; pa.N = p->n; pa.n_groups = p->n_adapters; pa.r = p->rank;
    pa.slots = L.m_pad;
    pa.route_blocks = routed ? 1u : 0u;
    pa.a_operand_steps = (p->k + 63u) / 64u; pa.a_operand_rb = rank_chunks(p->rank) > 2u ? 2u : 1u;  // lora_a_kernel's operand order
    const uint64_t a_items = (uint64_t)p->n_adapters * pa.a_operand_steps * pa.a_operand_rb * 256u;
    pa.a_blocks = (uint32_t)((a_items + 1023u) / 1024u);
    hipLaunchKernelGGL(lora_prep_kernel, dim3(pa.route_blocks + pa.a_blocks), dim3(1024), 0, s, pa);
    if ((st = launch_status())) return st;
    LoraAArgs la{};
    la.xsrc = q.x;
    la.at = at;
    la.at_operand = 1u;
    la.src_row = routed ? src_row : nullptr;
    la.slot_group = routed ? slot_group : nullptr;
    la.blk_range = routed ? blk_range : nullptr;
    la.zp = nullptr;
    la.zf = reinterpret_cast<float*>(ws + L.z);
    la.zf_stride = 64u;
    la.M = p->m; la.K = p->k; la.r = p->rank; la.nkk = rank_chunks(p->rank);
    const uint32_t nks = gq_z_ksplit(L.m_pad, p->k);
    la.n_steps = (p->k + 63u) / 64u; la.steps_per_wave = ((la.n_steps + nks - 1u) / nks + 15u) / 16u;
    la.n_ksplit = nks; la.zf_slice = L.m_pad * 64u;
    z_slices = nks; z_slice_stride = L.m_pad * 64u;
    la.nterms = 3u;
    la.n_blocks = L.m_pad / 32u;
    const dim3 zgrid(L.m_pad / 32u * nks), zblock(1024);
    (void)zblock;
    if ((st = launch_lora_a(la, la.nkk, zgrid, s))) return st;
  } else if (lora) {
    GqLoraZArgs z{};
    z.x = q.x;
    z.lora_a = static_cast<const uint16_t*>(p->lora_a);
    z.idx = p->adapter_indices;
    z.z = reinterpret_cast<float*>(ws + L.z);
    z.M = p->m; z.K = p->k; z.r = p->rank; z.n_adapters = p->n_adapters;
    z.k_split = decode ? (p->k + 255u) / 256u : 1u;
    if (z.k_split > kGqZSlices) z.k_split = kGqZSlices;
    z.k_chunk = round_up((p->k + z.k_split - 1u) / z.k_split, 64u);
    z_slices = z.k_split;
    const dim3 zgrid((p->m + 3u) / 4u, z.k_split), zblock(256);
    if (p->rank <= 8u) hipLaunchKernelGGL((gq_lora_z_kernel<1>), zgrid, zblock, 0, s, z);
    else if (p->rank <= 16u) hipLaunchKernelGGL((gq_lora_z_kernel<2>), zgrid, zblock, 0, s, z);
    else if (p->rank <= 32u) hipLaunchKernelGGL((gq_lora_z_kernel<4>), zgrid, zblock, 0, s, z);
    else hipLaunchKernelGGL((gq_lora_z_kernel<8>), zgrid, zblock, 0, s, z);
    if ((st = launch_status())) return st;
  }

  GqGemmArgs g{};
  g.codes = q.codes; g.xs = q.scales;
  g.wp = static_cast<const unsigned char*>(p->w_packed);
  g.ws = p->w_scales;
  g.z = lora ? reinterpret_cast<const float*>(ws + L.z) : nullptr;
  g.z_slot = routed ? dst_pos : nullptr;
  g.z_slices = z_slices; g.z_slice_stride = z_slice_stride;
  g.lora_b = static_cast<const uint16_t*>(p->lora_b);
  g.lora_scaling = p->lora_scaling;
  g.idx = p->adapter_indices;
  g.out = static_cast<uint16_t*>(p->out);
  g.aux_base = p->aux_base;
  g.M = p->m; g.M_pad = L.m_pad; g.N = p->n; g.K_pad = p->k_pad; g.group = p->group_size; g.G = L.G;
  g.bits = p->weight_bits;
  g.r = p->rank; g.n_adapters = p->n_adapters;
  g.n_col_blocks = (p->n + 31u) / 32u;
  if (L.m_pad == 32u) {  // decode: split the groups over the waves of a workgroup per column block
    const dim3 sgrid(g.n_col_blocks), sblock(kGqSkinnyWaves * 64u);
    if (p->weight_bits == 4u) hipLaunchKernelGGL((gq_skinny_kernel<true>), sgrid, sblock, 0, s, g);
    else hipLaunchKernelGGL((gq_skinny_kernel<false>), sgrid, sblock, 0, s, g);
    return launch_status();
  }
  if (p->group_size % 64u == 0 && !(p->flags & MI355_W8A8_FLAG_GQ_DIRECT)) {
    // groups of whole 64-wide k steps: 128 x 128 tiles staged through the LDS
    const dim3 grid((g.n_col_blocks + 3u) / 4u, (L.m_pad / 32u + 3u) / 4u), block(256);
    if (p->weight_bits == 4u) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gq_gemm_lds_kernel<true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gq_lds_bytes(true)) != hipSuccess)
        return MI355_W8A8_ERR_LAUNCH;
      hipLaunchKernelGGL((gq_gemm_lds_kernel<true>), grid, block, gq_lds_bytes(true), s, g);
    } else {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gq_gemm_lds_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gq_lds_bytes(false)) != hipSuccess)
        return MI355_W8A8_ERR_LAUNCH;
      hipLaunchKernelGGL((gq_gemm_lds_kernel<false>), grid, block, gq_lds_bytes(false), s, g);
    }
    return launch_status();
  }
  const dim3 grid((g.n_col_blocks + 7u) / 8u, (L.m_pad / 32u + 1u) / 2u), block(256);
  if (p->weight_bits == 4u) hipLaunchKernelGGL((gq_gemm_kernel<true>), grid, block, 0, s, g);
  else hipLaunchKernelGGL((gq_gemm_kernel<false>), grid, block, 0, s, g);
  return launch_status();
}

}  // namespace

extern "C" {

int mi355_w8a8_abi_version(void) { return MI355_W8A8_ABI_VERSION; }

const char* mi355_w8a8_status_string(int status) {
  switch (status) {
    case MI355_W8A8_OK: return "ok";
    case MI355_W8A8_ERR_NULL: return "a required pointer is NULL";
    case MI355_W8A8_ERR_SHAPE: return "a dimension or flag combination is invalid";
    case MI355_W8A8_ERR_ALIGN: return "a pointer is not sufficiently aligned";
    case MI355_W8A8_ERR_ALIAS: return "the output overlaps an input or the workspace";
    case MI355_W8A8_ERR_WORKSPACE: return "workspace missing or too small";
    case MI355_W8A8_ERR_LAUNCH: return "the HIP runtime refused a launch";
    case MI355_W8A8_ERR_UNSUPPORTED: return "request outside the supported geometry";
    case MI355_W8A8_ERR_STRUCT: return "struct_size does not match this library";
    default: return "unknown status";
  }
}

uint64_t mi355_w8a8_packed_weight_bytes(uint32_t k, uint32_t n) {
  if (k == 0 || n == 0) return 0;
  return (uint64_t)k_padded(k) * n_padded(n);
}

int mi355_w8a8_pack_weight_v1(const int8_t* codes_kn, void* packed, uint32_t k, uint32_t n, void* stream) {
  if (!codes_kn || !packed) return MI355_W8A8_ERR_NULL;
  if (k == 0 || n == 0) return MI355_W8A8_ERR_SHAPE;
  if (n > kMaxN || k > (1u << 20)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (!aligned16(packed)) return MI355_W8A8_ERR_ALIGN;
  const uint64_t bytes = mi355_w8a8_packed_weight_bytes(k, n);
  if (overlaps(codes_kn, (uint64_t)k * n, packed, bytes)) return MI355_W8A8_ERR_ALIAS;
  const uint64_t chunks = bytes / 16u;
  (void)hipGetLastError();
  hipLaunchKernelGGL(pack_weight_kernel, dim3((uint32_t)((chunks + 255u) / 256u)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), codes_kn, static_cast<unsigned char*>(packed), k, n,
                     k_padded(k) / 32u, chunks);
  return launch_status();
}

int mi355_w8a8_unpack_weight_v1(const void* packed, int8_t* codes_kn, uint32_t k, uint32_t n, void* stream) {
  if (!codes_kn || !packed) return MI355_W8A8_ERR_NULL;
  if (k == 0 || n == 0) return MI355_W8A8_ERR_SHAPE;
  if (n > kMaxN || k > (1u << 20)) return MI355_W8A8_ERR_UNSUPPORTED;
  if (overlaps(codes_kn, (uint64_t)k * n, packed, mi355_w8a8_packed_weight_bytes(k, n)))
    return MI355_W8A8_ERR_ALIAS;
  const uint64_t total = (uint64_t)k * n;
  (void)hipGetLastError();
  hipLaunchKernelGGL(unpack_weight_kernel, dim3((uint32_t)((total + 255u) / 256u)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const unsigned char*>(packed), codes_kn, k, n,
                     k_padded(k) / 32u);
  return launch_status();
}

int mi355_w8a8_quantize_rows_v1(const void* x_bf16, int8_t* codes, float* scales, uint32_t m, uint32_t k,
                                void* stream) {
  if (!x_bf16 || !codes || !scales) return MI355_W8A8_ERR_NULL;
  int st = validate_common(m, k, 1);
  if (st) return st;
  if (!aligned16(x_bf16) || (reinterpret_cast<uintptr_t>(codes) & 7u) || (reinterpret_cast<uintptr_t>(scales) & 3u))
    return MI355_W8A8_ERR_ALIGN;
  if (overlaps(x_bf16, (uint64_t)m * k * 2u, codes, (uint64_t)m * k) ||
      overlaps(x_bf16, (uint64_t)m * k * 2u, scales, (uint64_t)m * 4u) ||
      overlaps(codes, (uint64_t)m * k, scales, (uint64_t)m * 4u))
    return MI355_W8A8_ERR_ALIAS;
  QuantArgs q{};
  q.x = static_cast<const uint16_t*>(x_bf16);
  q.M = m; q.K = k; q.K_pad = k_padded(k); q.KB = q.K_pad / 32u;
  q.codes_rm = codes;
  q.scales_rm = scales;
  (void)hipGetLastError();
  return launch_quant<false>(q, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_adapters, uint32_t rank,
                                    uint32_t flags) {
  (void)flags;
  if (validate_common(m, k, n)) return 0;
  if (n_adapters > (uint32_t)kMaxAdapters || rank > (uint32_t)kMaxRank) return 0;
  // (sized for groups on block boundaries wherever a call of these dimensions may lay them out so)
  return make_layout(m, k, n, n_adapters, n_adapters ? rank : 0u, n_adapters > 1,
                     padded_groups_fit(m, n, n_adapters) || padded_groups_fit(m, n, n_adapters, true)).total;
}

int mi355_w8a8_lora_linear_v1(const mi355_w8a8_problem* p, void* stream) {
  return run_forward(p, static_cast<hipStream_t>(stream), kReqLinear);
}
int mi355_w8a8_rms_gateup_swiglu_v1(const mi355_w8a8_problem* p, void* stream) {
  return run_forward(p, static_cast<hipStream_t>(stream), kReqGateUp);
}
int mi355_w8a8_lora_residual_v1(const mi355_w8a8_problem* p, void* stream) {
  return run_forward(p, static_cast<hipStream_t>(stream), kReqResidual);
}
int mi355_w8a8_forward_v1(const mi355_w8a8_problem* p, void* stream) {
  return run_forward(p, static_cast<hipStream_t>(stream), kReqNone);
}

int mi355_w8a8_forward_static_ws_v1(const mi355_w8a8_problem* p, void* stream) {
  if (!p) return MI355_W8A8_ERR_NULL;
  if (p->struct_size != sizeof(mi355_w8a8_problem)) return MI355_W8A8_ERR_STRUCT;
  const int st = validate_common(p->m, p->k, p->n);
  if (st) return st;
  // Every caller in the process shares the array: what an earlier call left in it may be another layer's,
  // so a call must not be told to keep it.
  if (p->flags & (MI355_W8A8_FLAG_LORA_PACK_VALID | MI355_W8A8_FLAG_SKIP_PROLOGUE)) return MI355_W8A8_ERR_UNSUPPORTED;
  const uint64_t need = mi355_w8a8_workspace_bytes(p->m, p->k, p->n, p->n_adapters, p->rank, p->flags);
  if (need == 0 || need > MI355_W8A8_STATIC_WORKSPACE_BYTES) return MI355_W8A8_ERR_WORKSPACE;
  void* ws = static_workspace();
  if (!ws) return MI355_W8A8_ERR_LAUNCH;
  // Nothing in the workspace has to start at zero: every table a kernel reads is written by an earlier
  // kernel of the same call (the tile counters are cleared by the quantizer launch), so the contents a
  // previous call left behind are never read.
  mi355_w8a8_problem q = *p;
  q.workspace = ws;
  q.workspace_bytes = MI355_W8A8_STATIC_WORKSPACE_BYTES;
  return run_forward(&q, static_cast<hipStream_t>(stream), kReqNone);
}

uint64_t mi355_w8a8_grouped_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank,
                                            uint32_t flags) {
  if (validate_common(m, k, n)) return 0;
  if (n_groups == 0 || n_groups > (uint32_t)kMaxGroups || rank > (uint32_t)kMaxRank) return 0;
  return make_grouped_layout(m, k, n, n_groups, rank, flags).total;
}

int mi355_w8a8_grouped_v1(const mi355_w8a8_grouped_problem* p, void* stream) {
  return run_grouped(p, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_bwd_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_adapters, uint32_t rank,
                                        uint32_t flags) {
  (void)flags;
  if (validate_bwd_dims(m, k, n, n_adapters, rank)) return 0;
  return make_bwd_layout(m, k, n, n_adapters, n_adapters ? rank : 0u).total;
}

int mi355_w8a8_lora_linear_bwd_v1(const mi355_w8a8_bwd_problem* p, void* stream) {
  return run_backward(p, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_grouped_bwd_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups, uint32_t rank,
                                                uint32_t groups_per_weight) {
  if (validate_bwd_grouped_dims(m, k, n, n_groups, rank, groups_per_weight)) return 0;
  return make_bwd_grouped_layout(m, k, n, n_groups, rank, groups_per_weight).total;
}

int mi355_w8a8_grouped_bwd_v1(const mi355_w8a8_grouped_bwd_problem* p, void* stream) {
  return run_grouped_backward(p, static_cast<hipStream_t>(stream));
}

int mi355_w8a8_qkv_split_norm_rope_v1(const mi355_w8a8_qkv_post_problem* p, void* stream) {
  return run_qkv_post(p, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_qkv_bwd_workspace_bytes(uint32_t m, uint32_t head_dim) { return qkv_bwd_workspace_bytes(m, head_dim); }

int mi355_w8a8_qkv_split_norm_rope_bwd_v1(const mi355_w8a8_qkv_post_bwd_problem* p, void* stream) {
  return run_qkv_post_bwd(p, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_delta_rms_norm_bwd_workspace_bytes(uint32_t m, uint32_t k) {
  return delta_rms_bwd_workspace_bytes(m, k);
}

int mi355_w8a8_delta_rms_norm_bwd_v1(const void* x, const float* gamma, const void* d_normalized, void* d_x,
                                     float* d_gamma, void* workspace, uint64_t workspace_bytes, uint32_t m,
                                     uint32_t k, float eps, void* stream) {
  return run_delta_rms_norm_bwd(x, gamma, d_normalized, d_x, d_gamma, workspace, workspace_bytes, m, k, eps,
                                static_cast<hipStream_t>(stream));
}

int mi355_w8a8_swiglu_v1(const void* fused, void* product, uint32_t m, uint32_t n, void* stream) {
  return run_swiglu_fwd(fused, product, m, n, static_cast<hipStream_t>(stream));
}

int mi355_w8a8_swiglu_bwd_v1(const void* fused, const void* d_product, void* d_fused, uint32_t m, uint32_t n,
                             void* stream) {
  return run_swiglu_bwd(fused, d_product, d_fused, m, n, static_cast<hipStream_t>(stream));
}

int mi355_w8a8_rms_norm_bwd_v1(const void* x, const float* gamma, const void* d_normalized, void* d_x, uint32_t m,
                               uint32_t k, float eps, void* stream) {
  return run_rms_norm_bwd(x, gamma, d_normalized, d_x, m, k, eps, static_cast<hipStream_t>(stream));
}

int mi355_w8a8_moe_route_v1(const float* router_logits, uint32_t n_tokens, uint32_t n_experts, uint32_t top_k,
                            uint32_t norm_topk_prob, float* weights, int32_t* selected, void* stream) {
  return run_moe_route(router_logits, n_tokens, n_experts, top_k, norm_topk_prob, weights, selected,
                       static_cast<hipStream_t>(stream));
}

int mi355_w8a8_moe_route_bwd_v1(const float* router_logits, const int32_t* selected, const float* d_weights,
                                uint32_t n_tokens, uint32_t n_experts, uint32_t top_k, uint32_t norm_topk_prob,
                                float* d_router_logits, void* stream) {
  return run_moe_route_bwd(router_logits, selected, d_weights, n_tokens, n_experts, top_k, norm_topk_prob,
                           d_router_logits, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_moe_dispatch_workspace_bytes(uint32_t n_pairs, uint32_t n_groups) {
  if (validate_moe_sort_dims(n_pairs, n_groups)) return 0;
  return make_moe_sort_layout(n_pairs, n_groups).total;
}

int mi355_w8a8_moe_dispatch_v1(const mi355_w8a8_moe_dispatch_problem* p, void* stream) {
  return run_moe_dispatch(p, static_cast<hipStream_t>(stream));
}

int mi355_w8a8_moe_combine_v1(const void* expert_out, const int32_t* unsort_indices, const float* weights, void* out,
                              uint32_t n_tokens, uint32_t top_k, uint32_t width, void* stream) {
  return run_moe_combine(expert_out, unsort_indices, weights, out, n_tokens, top_k, width,
                         static_cast<hipStream_t>(stream));
}

int mi355_w8a8_moe_combine_bwd_v1(const void* d_out, const void* expert_out, const int32_t* sort_indices,
                                  const float* weights, void* d_expert_out, float* d_weights, uint32_t n_tokens,
                                  uint32_t top_k, uint32_t width, void* stream) {
  return run_moe_combine_bwd(d_out, expert_out, sort_indices, weights, d_expert_out, d_weights, n_tokens, top_k, width,
                             static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_gq_packed_weight_bytes(uint32_t k_pad, uint32_t n, uint32_t weight_bits) {
  if (k_pad == 0 || (k_pad & 31u) || n == 0 || (weight_bits != 4u && weight_bits != 8u)) return 0;
  return gq_packed_bytes(k_pad, n, weight_bits);
}

int mi355_w8a8_gq_pack_weight_v1(const void* codes, void* packed, uint32_t k_pad, uint32_t n, uint32_t weight_bits,
                                 void* stream) {
  return run_gq_pack(codes, packed, k_pad, n, weight_bits, static_cast<hipStream_t>(stream));
}

uint64_t mi355_w8a8_gq_workspace_bytes(uint32_t m, uint32_t k_pad, uint32_t group_size, uint32_t n_adapters,
                                       uint32_t rank) {
  if (validate_gq_dims(m, k_pad, group_size, rank)) return 0;
  return make_gq_layout(m, k_pad, group_size, n_adapters, n_adapters ? rank : 0u).total;
}

int mi355_w8a8_gq_linear_v1(const mi355_w8a8_gq_problem* p, void* stream) {
  return run_gq_linear(p, static_cast<hipStream_t>(stream));
}

int mi355_w8a8_forward_path(uint32_t m, uint32_t k, uint32_t n, uint32_t flags) {
  const int st = validate_common(m, k, n);
  if (st) return st;
  if ((flags & MI355_W8A8_FLAG_FORCE_TILED) && (flags & MI355_W8A8_FLAG_FORCE_SKINNY)) return MI355_W8A8_ERR_SHAPE;
  return choose_forward_path(m, k, n, flags);
}

uint64_t mi355_w8a8_calibrate_operand_bytes(void) { return kCalOperandBytes; }

uint64_t mi355_w8a8_calibrate_mfma_ops(uint32_t shape, uint32_t iters) {
  // per wave and round: 16 x (2 x 32 x 32 x 32) or 64 x (2 x 16 x 16 x 64) operations; 4 waves x 256 workgroups
  if (shape > 1u) return 0;
  return (shape == 1u ? 64ull * 32768ull : 16ull * 65536ull) * 4ull * kCalGrid * iters;
}

int mi355_w8a8_calibrate_mfma_v1(uint32_t shape, const void* operands, uint32_t iters, uint64_t* clocks,
                                 int32_t* sink, void* stream) {
  if (!operands || !clocks || !sink) return MI355_W8A8_ERR_NULL;
  if (shape > 1u || iters == 0 || iters > (1u << 18)) return MI355_W8A8_ERR_SHAPE;  // (2^18 rounds keep a launch under half a second)
  if (reinterpret_cast<uintptr_t>(operands) & 15u) return MI355_W8A8_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned char* src = static_cast<const unsigned char*>(operands);
  if (shape == 1u) hipLaunchKernelGGL(cal_mfma_kernel<1>, dim3(kCalGrid), dim3(256), 0, s, src, iters, clocks, sink);
  else hipLaunchKernelGGL(cal_mfma_kernel<0>, dim3(kCalGrid), dim3(256), 0, s, src, iters, clocks, sink);
  return launch_status();
}

int mi355_w8a8_calibrate_read_v1(const void* src, uint64_t bytes, uint32_t* sink, void* stream) {
  if (!src || !sink) return MI355_W8A8_ERR_NULL;
  if (bytes == 0 || (bytes & 32767u)) return MI355_W8A8_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(src) & 15u) return MI355_W8A8_ERR_ALIGN;
  hipLaunchKernelGGL(cal_read_kernel, dim3(2048), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const v4i*>(src), bytes / 16u, sink);
  return launch_status();
}

int mi355_w8a8_calibrate_copy_v1(const void* src, void* dst, uint64_t bytes, void* stream) {
  if (!src || !dst) return MI355_W8A8_ERR_NULL;
  if (bytes == 0 || (bytes & 15u)) return MI355_W8A8_ERR_SHAPE;
  if (!aligned16(src) || !aligned16(dst)) return MI355_W8A8_ERR_ALIGN;
  if (overlaps(src, bytes, dst, bytes)) return MI355_W8A8_ERR_ALIAS;
  hipLaunchKernelGGL(cal_copy_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const v4i*>(src), static_cast<v4i*>(dst), bytes / 16u);
  return launch_status();
}

}  // extern "C"
