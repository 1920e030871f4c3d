// bf16 MFMA kernels for gfx950 (v_mfma_f32_32x32x16_bf16): weight packing and the token-tile-major fused
// experts kernel (up-projection + bias + activation + routing mask + down-projection, nothing spilled to HBM).
//
// Fragment layouts of the 32x32x16 bf16 MFMA on a 64-lane wave (g = lane / 32, c = lane % 32):
//   A (32 x 16): lane holds row c,    k = 8g .. 8g+7      (8 bf16 = 16 bytes)
//   B (16 x 32): lane holds column c, k = 8g .. 8g+7
//   C (32 x 32): lane holds column c, rows 8*(r/4) + 4g + (r%4) for r = 0..15
//
// The fused kernel computes the first GEMM transposed (H^T = W1^T . X^T), so a lane ends up holding, for ONE
// token (column c), 16 hidden neurons.  Read as an A fragment of the second GEMM (row = token, k = hidden) those
// registers are already in place: r = 0..7 feed one K=16 step, r = 8..15 the next.  The k-slot -> hidden-neuron
// map this implies (slot (g, i) of a step <-> neuron 8*(i/4) + 4g + (i%4) of a 16-block) is baked into the
// packed W2 fragments, so no shuffle is needed between the two GEMMs.
#include "dense_sweep.hpp"

namespace d2dmoe {

size_t dense_lds_bytes(const d2dmoe_shape& sh) {
  const int hc = sweep_chunk(sh.d_model);
  const int hidden = sh.n_experts * sh.expert_dim;
  const int n_chunks = (hidden + hc - 1) / hc;
  const int KS1 = sh.d_model / 16;
  return (size_t)(2 * KS1 * 64 + 2 * (hc / 16) * 64) * 16         // x fragments, h fragments
         + (sh.d_model <= 768 ? (size_t)MD_BM * (sh.n_experts + 8) * 2 : 0)   // routing tile, rows padded by 8 elements
         + (size_t)n_chunks * hc * 3                               // b1 (bf16) and expert index (uint8) per neuron
         + (size_t)((sh.n_experts + 7) / 8 * 8 + 4) * sizeof(uint32_t)    // per expert: chunk bits (fixed chunks) or one bit per expert (gathered); the active-chunk mask
         + (size_t)MD_WAVES * MD_MAX_CHUNKS * 8;                            // every wave's list of blocks
}

// The fused experts kernel is instantiated for D = 768 (ViT-B, GPT-2 small, BERT-base) and D = 1024 (GPT-2 medium,
// BERT-large, ViT-L), ungated experts, bf16 and float16.
bool mfma_dense_supported(const d2dmoe_shape& sh) {
  if ((sh.dtype != D2DMOE_BF16 && sh.dtype != D2DMOE_F16) || sh.gated) return false;
  if (sh.d_model != 768 && sh.d_model != 1024) return false;
  const int hc = sweep_chunk(sh.d_model);
  if (sh.n_experts > 256) return false;          // expert indices are staged as uint8
  if (sh.expert_dim > hc) return false;          // an expert spans at most two chunks
  if ((sh.n_experts * sh.expert_dim + hc - 1) / hc > MD_MAX_CHUNKS) return false;   // staging registers, chunk mask
  return dense_lds_bytes(sh) <= 160 * 1024;      // x tile + h tile (+ routing tile) + bias/expert-index tables
}

// The expert-major path hands over to the sweep on the device wherever there is one; else to the tiled products.
bool mfma_sparse_falls_back_to_sweep(const d2dmoe_shape& sh) { return !sh.gated && mfma_dense_supported(sh); }

// The fused router+select kernel covers the D2DMoE router: bf16, depth 2, ReLU hidden / abs output activation,
// width and expert count both 128 or both 256, D a multiple of 64.
bool mfma_router_supported(const d2dmoe_shape& sh) {
  if ((sh.dtype != D2DMOE_BF16 && sh.dtype != D2DMOE_F16) || sh.router_width <= 0) return false;
  if (sh.router_activation != D2DMOE_ACT_RELU || sh.router_output_activation != D2DMOE_ACT_ABS) return false;
  if (sh.d_model % 64 != 0) return false;
  // hidden widths 128 and 256; any number of experts that keeps rows of the routing matrix 16-byte aligned, up to 256
  // (the second product works on tiles of 32 experts: the packed W2 is padded with zero rows)
  if (sh.router_width != 128 && sh.router_width != 256) return false;
  return sh.n_experts % 8 == 0 && sh.n_experts >= 8 && sh.n_experts <= 256;
}

// experts the router kernels compute on: a multiple of 32 they are instantiated for
int mfma_router_padded_experts(const d2dmoe_shape& sh) {
  if (sh.router_width == 256) return 256;
  return sh.n_experts <= 32 ? 32 : (sh.n_experts <= 64 ? 64 : (sh.n_experts <= 128 ? 128 : 256));
}

// the shapes the resident and the split kernels are written for (the others run the one-wave-per-tile kernel)
static bool router_shape_exact(const d2dmoe_shape& sh) {
  return (sh.router_width == 128 && sh.n_experts == 128) || (sh.router_width == 256 && sh.n_experts == 256);
}

// The expert-major kernel covers the same layers as the dense sweep with experts of at most 128 neurons.
// Gated experts have their own expert-major kernel, instantiated for D = 2048 and experts of at most 64 neurons (Gemma).
bool mfma_sparse_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 && sh.dtype != D2DMOE_F16) return false;
  if (sh.gated) return sh.d_model == 2048 && sh.expert_dim <= 64 && sh.n_experts <= 1024;
  if (sh.n_experts > 1024) return false;
  if (sh.d_model == 768) return sh.expert_dim <= 128;
  // wider models: the registers a wave needs grow with D and with the expert's row tiles
  if (sh.d_model == 1024) return sh.expert_dim <= 64;
  if (sh.d_model == 1280) return sh.expert_dim <= 32;
  return false;
}

PackedLayout packed_layout(const d2dmoe_shape& sh) {
  PackedLayout L;
  L.hidden = sh.n_experts * sh.expert_dim;
  const int hc = sweep_chunk(sh.d_model);
  L.n_chunks = (L.hidden + hc - 1) / hc;
  L.hidden_pad = L.n_chunks * hc;
  L.pieces = sh.d_model / 16 * (hc / 128) + (hc / 16) * (sh.d_model / 128);
  size_t off = PACKED_HEADER_BYTES;   // the buffer starts with its descriptor
  L.has_dense = mfma_dense_supported(sh);
  L.w_off = off;    if (L.has_dense) off += (size_t)MD_WAVES * L.n_chunks * L.pieces * 64 * 16;
  L.b1_off = off;   if (L.has_dense) off += (size_t)L.hidden_pad * 2;   // bf16
  L.eidx_off = off; if (L.has_dense) off += (size_t)L.hidden_pad;       // uint8
  off = (off + 255) / 256 * 256;
  L.has_sparse = mfma_sparse_supported(sh);
  const int nt = (sh.expert_dim + 31) / 32;
  L.nt = (nt <= 1) ? 1 : (nt == 2 ? 2 : 4);   // kernels are instantiated for 1, 2 and 4 row tiles
  if (sh.gated) L.nt = 2;                      // the gated kernel always works on two tiles per projection
  const size_t frag_bytes = (size_t)sh.n_experts * L.nt * 32 * sh.d_model * 2;
  L.s1_off = off;   if (L.has_sparse) off += frag_bytes;
  L.su_off = off;   if (L.has_sparse && sh.gated) off += frag_bytes;
  L.s2_off = off;   if (L.has_sparse) off += frag_bytes;
  L.sb_off = off;   if (L.has_sparse) off += (size_t)sh.n_experts * L.nt * 32 * 2;
  off = (off + 255) / 256 * 256;
  L.has_decode = mfma_decode_supported(sh);
  L.dc_off = off;   if (L.has_decode) off += mfma_decode_packed_bytes(sh);
  L.has_gemm = mfma_gemm_supported(sh);
  L.gm_off = off;   if (L.has_gemm) off += mfma_gemm_packed_bytes(sh);
  L.has_mid = mfma_mid_supported(sh);     // experts padded to 32 neurons, both layers
  const size_t mid_bytes = (size_t)sh.n_experts * MID_HROW * sh.d_model * 2;
  L.m1_off = off;   if (L.has_mid) off += mid_bytes;
  L.m2_off = off;   if (L.has_mid) off += mid_bytes;
  // the router section comes last, so the expert sections sit at the same offsets whether or not the shape handed
  // to a later call names the router
  L.has_router = mfma_router_supported(sh);
  L.r1_off = off;   if (L.has_router) off += (size_t)sh.router_width * sh.d_model * 2;
  L.r2_off = off;   if (L.has_router) off += (size_t)mfma_router_padded_experts(sh) * sh.router_width * 2;
  L.total = (off + 255) / 256 * 256;
  if (!(L.has_dense || L.has_sparse || L.has_decode || L.has_gemm || L.has_mid || L.has_router)) L.total = 0;
  return L;
}

size_t mfma_packed_bytes(const d2dmoe_shape& sh) { return packed_layout(sh).total; }

unsigned mfma_packed_sections(const d2dmoe_shape& sh) {
  const PackedLayout L = packed_layout(sh);
  return (L.has_dense ? D2DMOE_SECTION_DENSE : 0u) | (L.has_sparse ? D2DMOE_SECTION_EXPERT_MAJOR : 0u) |
         (L.has_decode ? D2DMOE_SECTION_SMALL_BATCH : 0u) | (L.has_gemm ? D2DMOE_SECTION_TILED : 0u) |
         (L.has_mid ? D2DMOE_SECTION_COMPACTED : 0u) | (L.has_router ? D2DMOE_SECTION_ROUTER : 0u);
}

// The descriptor's 64 bytes at the start of the buffer (for a caller that wants to recover it from the buffer).
__global__ void pack_header_kernel(const d2dmoe_packed_desc d, d2dmoe_packed_desc* dst) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *dst = d;
}

hipError_t launch_pack_header(const d2dmoe_packed_desc& d, void* packed, hipStream_t s) {
  hipLaunchKernelGGL(pack_header_kernel, dim3(1), dim3(64), 0, s, d, (d2dmoe_packed_desc*)packed);
  return hipGetLastError();
}
size_t mfma_decode_section_offset(const d2dmoe_shape& sh) { return packed_layout(sh).dc_off; }
size_t mfma_gemm_section_offset(const d2dmoe_shape& sh) { return packed_layout(sh).gm_off; }

// ---------------------------------------------------------------------------------------------------
// Packing.  Each wave of the fused kernel reads ONE linear stream of 1 KB fragments (16 bytes per lane), in the
// order the kernel consumes them:
//   stream[wave][chunk][piece][lane][8 bf16],   KS1 = D/16, CT = D/128, HC = neurons per chunk, RT = HC/128, KS2 = HC/16
//   pieces [0, RT KS1)         W1 fragments, piece = kstep*RT + rt:
//       neuron h = chunk*HC + wave*32*RT + rt*32 + c,  d = kstep*16 + 8g + i      value w1[h/Ed][d][h%Ed]
//   pieces [RT KS1, RT KS1 + KS2 CT) W2 fragments, piece = RT KS1 + ks2*CT + ct:
//       neuron h = chunk*HC + (ks2/2)*32 + (ks2%2)*16 + 8*(i/4) + 4g + (i%4)
//       column   = wave*(D/4) + ct*32 + c                                         value w2[h/Ed][h%Ed][column]
// plus b1 as bf16 [hidden_pad] and the expert index of every neuron as uint8 [hidden_pad]; padding neurons
// (beyond E*Ed) carry zero weights and zero bias.  One thread per 16-byte piece.
// ---------------------------------------------------------------------------------------------------
__global__ void pack_stream_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ w2, bf16_t* __restrict__ dst,
                                   int D, int Ed, int hidden, int n_chunks, int pieces, int64_t n_items) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_items) return;
  const int lane = (int)(p % 64);
  int64_t q = p / 64;
  const int piece = (int)(q % pieces); q /= pieces;
  const int chunk = (int)(q % n_chunks);
  const int wave = (int)(q / n_chunks);
  const int g = lane / 32, c = lane % 32;
  const int KS1 = D / 16, CT = D / 128;
  const int HC = sweep_chunk(D), RT = HC / 128;
  bf16_t v[8];
  if (piece < RT * KS1) {
    const int ks = piece / RT, rt = piece % RT;
    const int h = chunk * HC + wave * 32 * RT + rt * 32 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 16 + 8 * g + i;
      v[i] = (h < hidden) ? w1[((int64_t)(h / Ed) * D + d) * Ed + (h % Ed)] : (bf16_t)0;
    }
  } else {
    const int r = piece - RT * KS1;
    const int ks2 = r / CT, ct = r % CT;
    const int col = wave * (D / 4) + ct * 32 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int h = chunk * HC + (ks2 / 2) * 32 + (ks2 % 2) * 16 + 8 * (i / 4) + 4 * g + (i % 4);
      v[i] = (h < hidden) ? w2[((int64_t)(h / Ed) * Ed + (h % Ed)) * D + col] : (bf16_t)0;
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) dst[p * 8 + i] = v[i];
}

__global__ void pack_bias_kernel(const bf16_t* __restrict__ b1, bf16_t* __restrict__ b1p, uint8_t* __restrict__ eidx,
                                 int Ed, int hidden, int hidden_pad) {
  const int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= hidden_pad) return;
  b1p[h] = (h < hidden && b1 != nullptr) ? b1[h] : (bf16_t)0;
  eidx[h] = (uint8_t)((h < hidden) ? (h / Ed) : 0);
}

// Router fragments.
//   W1 fragments [kstep D/16][row-tile W/32][lane][8]:  row w = rt*32 + c, d = kstep*16 + 8g + i     value W1[w][d]
//   W2 fragments [kstep2 W/16][row-tile E/32][lane][8]: row e = et*32 + c,
//       w = (ks2/2)*32 + (ks2%2)*16 + 8*(i/4) + 4g + (i%4)  (the k order in which the first GEMM leaves the hidden
//       activations in registers)                                                                   value W2[e][w]
__global__ void pack_router_kernel(const bf16_t* __restrict__ rw1, const bf16_t* __restrict__ rw2, bf16_t* __restrict__ d1,
                                   bf16_t* __restrict__ d2, int D, int W, int E, int e_real) {   // E: padded to tiles of 32
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n1 = (int64_t)W * D / 8, n2 = (int64_t)E * W / 8;
  const int lane = (int)(p % 64);
  const int g = lane / 32, c = lane % 32;
  if (p < n1) {
    const int WT = W / 32;
    const int64_t q = p / 64;
    const int rt = (int)(q % WT), ks = (int)(q / WT);
#pragma unroll
    for (int i = 0; i < 8; ++i) d1[p * 8 + i] = rw1[(int64_t)(rt * 32 + c) * D + ks * 16 + 8 * g + i];
  } else if (p < n1 + n2) {
    const int64_t pp = p - n1;
    const int ET = E / 32;
    const int64_t q = pp / 64;
    const int et = (int)(q % ET), ks2 = (int)(q / ET);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int wi = (ks2 / 2) * 32 + (ks2 % 2) * 16 + 8 * (i / 4) + 4 * g + (i % 4);
      d2[pp * 8 + i] = (et * 32 + c < e_real) ? rw2[(int64_t)(et * 32 + c) * W + wi] : (bf16_t)0;
    }
  }
}

hipError_t launch_mfma_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            const void* router_w1, const void* router_w2, void* packed, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  char* base = (char*)packed;
  if (L.has_router) {
    if (router_w1 == nullptr || router_w2 == nullptr) return hipErrorInvalidValue;
    const int e_pad = mfma_router_padded_experts(sh);
    const int64_t n = ((int64_t)sh.router_width * sh.d_model + (int64_t)e_pad * sh.router_width) / 8;
    hipLaunchKernelGGL(pack_router_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)router_w1,
                       (const bf16_t*)router_w2, (bf16_t*)(base + L.r1_off), (bf16_t*)(base + L.r2_off), sh.d_model,
                       sh.router_width, e_pad, sh.n_experts);
  }
  if (L.has_sparse) {
    hipError_t e = launch_sparse_pack(sh, L, w1, b1, w2, w_up, packed, s);
    if (e != hipSuccess) return e;
  }
  if (L.has_decode) {
    hipError_t e = launch_decode_pack(sh, w1, b1, w2, w_up, base + L.dc_off, s);
    if (e != hipSuccess) return e;
  }
  if (L.has_gemm) {
    hipError_t e = launch_gemm_pack(sh, w1, b1, w2, w_up, base + L.gm_off, s);
    if (e != hipSuccess) return e;
  }
  if (L.has_mid) {
    hipError_t e = launch_mid_pack(sh, L, w1, w2, packed, s);
    if (e != hipSuccess) return e;
  }
  if (!L.has_dense) return hipGetLastError();
  const int64_t n_items = (int64_t)MD_WAVES * L.n_chunks * L.pieces * 64;
  const unsigned blocks = (unsigned)((n_items + 255) / 256);
  hipLaunchKernelGGL(pack_stream_kernel, dim3(blocks), dim3(256), 0, s, (const bf16_t*)w1, (const bf16_t*)w2,
                     (bf16_t*)(base + L.w_off), sh.d_model, sh.expert_dim, L.hidden, L.n_chunks, L.pieces, n_items);
  hipLaunchKernelGGL(pack_bias_kernel, dim3((L.hidden_pad + 255) / 256), dim3(256), 0, s, (const bf16_t*)b1,
                     (bf16_t*)(base + L.b1_off), (uint8_t*)(base + L.eidx_off), sh.expert_dim, L.hidden, L.hidden_pad);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Fused experts kernel, token-tile-major ("masked dense sweep"): the kernels are templates in dense_sweep.hpp; here
// their tiling and the D = 768 instances.
// ---------------------------------------------------------------------------------------------------
int device_cu_count() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
    return cus;
  }();
  return n;
}


// Tiles of 64 tokens fill whole rounds of one workgroup per CU.  When the last round would be at most half full its
// tokens go to tiles of 32 instead, and if those still leave CUs idle each of them is dealt to several workgroups by
// chunk ranges -- so the tail of the launch (or, with few tokens, the whole launch) spreads over the machine.
DenseTiling dense_tiling(const d2dmoe_shape& sh, bool allow_split) {
  const int cus = device_cu_count();
  const int hc = sweep_chunk(sh.d_model);
  const int n_chunks = (sh.n_experts * sh.expert_dim + hc - 1) / hc;
  DenseTiling T;
  const int64_t t64 = cdiv64(sh.n_tokens, 64);
  const int64_t leftover = t64 % cus;
  T.n_full = t64; T.n_half = 0;
  T.csplit = 1; T.per = n_chunks; T.part_base = 0; T.part_rows = 0;
  if (leftover > 0 && leftover * 2 <= cus) {
    T.n_full = t64 - leftover;
    T.n_half = cdiv64(sh.n_tokens - T.n_full * 64, 32);
    if (allow_split && n_chunks >= 2 && T.n_half * 2 <= cus) {
      int cs = (int)(cus / T.n_half);
      if (cs > n_chunks) cs = n_chunks;
      T.per = (n_chunks + cs - 1) / cs;
      T.csplit = (n_chunks + T.per - 1) / T.per;
      if (T.csplit > 1) {
        T.part_base = T.n_full * 64;
        T.part_rows = sh.n_tokens - T.part_base;
      } else {
        T.per = n_chunks;
      }
    }
  }
  return T;
}

size_t mfma_dense_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_dense_supported(sh) || sh.n_tokens <= 0) return 0;
  const DenseTiling T = dense_tiling(sh, true);
  return T.csplit > 1 ? (size_t)T.csplit * T.part_rows * sh.d_model * 4 : 0;
}

hipError_t launch_mfma_dense(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                             const void* last_bias, void* out, const int* skip_flag, void* workspace, size_t workspace_bytes,
                             hipStream_t s) {
  if (sh.d_model != 768) return launch_mfma_dense_wide(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
  switch (sh.activation) {
    case D2DMOE_ACT_RELU:
      return launch_dense_act<768, D2DMOE_ACT_RELU>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
    case D2DMOE_ACT_GELU:
      return launch_dense_act<768, D2DMOE_ACT_GELU>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
    default:
      return launch_dense_act<768, -1>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
  }
}

// ---------------------------------------------------------------------------------------------------
// Fused router MLP + dynamic-k selection (moefication.py:328-330 and :80-85).
// One wave owns 32 tokens end to end; nothing goes through LDS or HBM between the stages:
//   GEMM1  H1^T[W, 32 tokens] = W1 . X^T          A = W1 fragments, B = x read straight from its rows
//          relu, round to bf16 -> the accumulators already sit in B-fragment position for the next product
//   GEMM2  NORMS^T[E, 32 tokens] = W2 . H1^T       A = W2 fragments (k order matched at packing)
//          abs, round to bf16; per-token maximum = in-lane maximum + one cross-half exchange (NaN-propagating);
//          thr = bf16(max * thr_scale); routing = norms >= thr ? 1 : 0
// A lane ends up with one token and 4 consecutive experts per accumulator quad, stored as 8-byte pieces.
// Optional outputs: the norms, and per-expert token counts (wave ballots + one integer atomic per expert).
// ---------------------------------------------------------------------------------------------------
template <int WT, int ET, int U, bool F16 = false>
__global__ __launch_bounds__(256) void router_select_mfma_kernel(
    const bf16_t* __restrict__ x, const bf16x8* __restrict__ w1f, const bf16x8* __restrict__ w2f,
    bf16_t* __restrict__ routing, bf16_t* __restrict__ norms_out, int32_t* __restrict__ counts, int64_t N, int D,
    float thr_scale, int e_real) {   // e_real <= ET * 32 experts exist (a multiple of 8); the rest are zero rows of W2
  constexpr uint32_t ONE = F16 ? 0x3C00u : 0x3F80u;   // 1.0 in the storage type
  constexpr int E = ET * 32;
  __shared__ __attribute__((aligned(16))) unsigned char stage_all[4 * 32 * E * 2];   // per wave: 32 rows of routing
  const int lane = threadIdx.x & 63;
  const int g = lane >> 5, c32 = lane & 31;
  const int64_t tok0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 32;
  if (tok0 >= N) return;   // whole wave; the kernel has no barriers
  const int64_t token = tok0 + c32;
  const bool valid = token < N;
  const bf16x8* xrow = (const bf16x8*)(x + (valid ? token : (N - 1)) * D);
  const int KS1 = D / 16;   // a multiple of 4 (checked by the launcher's support test)

  f32x16 acc1[WT];
#pragma unroll
  for (int a = 0; a < WT; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[a][r] = 0.f;
  // two register buffers of U K steps each (x rows and W1 fragments): one is multiplied while the other fills;
  // KS1 is a multiple of 2*U (the launcher picks U that way)
  bf16x8 xA[U], wA[U][WT], xB[U], wB[U][WT];
  auto fill = [&](bf16x8 (&xb)[U], bf16x8 (&wr)[U][WT], int ks0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      xb[u] = xrow[2 * (ks0 + u) + g];
#pragma unroll
      for (int rt = 0; rt < WT; ++rt) wr[u][rt] = w1f[(int64_t)((ks0 + u) * WT + rt) * 64 + lane];
    }
  };
  auto multiply = [&](bf16x8 (&xb)[U], bf16x8 (&wr)[U][WT]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int rt = 0; rt < WT; ++rt) acc1[rt] = mfma_32x32x16<F16>(wr[u][rt], xb[u], acc1[rt]);
  };
  fill(xA, wA, 0);
  for (int ks0 = 0; ks0 < KS1; ks0 += 2 * U) {
    fill(xB, wB, ks0 + U);
    multiply(xA, wA);
    fill(xA, wA, (ks0 + 2 * U < KS1) ? (ks0 + 2 * U) : ks0);   // the last trip re-reads its own steps: in bounds, unused
    multiply(xB, wB);
  }
  // hidden activations as B fragments of the second product
  bf16x8 hb[2 * WT];
#pragma unroll
  for (int rt = 0; rt < WT; ++rt)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint4 pk;
      pk.x = enc16x2<F16>(fmaxf(acc1[rt][half * 8 + 0], 0.f), fmaxf(acc1[rt][half * 8 + 1], 0.f));
      pk.y = enc16x2<F16>(fmaxf(acc1[rt][half * 8 + 2], 0.f), fmaxf(acc1[rt][half * 8 + 3], 0.f));
      pk.z = enc16x2<F16>(fmaxf(acc1[rt][half * 8 + 4], 0.f), fmaxf(acc1[rt][half * 8 + 5], 0.f));
      pk.w = enc16x2<F16>(fmaxf(acc1[rt][half * 8 + 6], 0.f), fmaxf(acc1[rt][half * 8 + 7], 0.f));
      __builtin_memcpy(&hb[rt * 2 + half], &pk, 16);
    }
  f32x16 acc2[ET];
#pragma unroll
  for (int a = 0; a < ET; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc2[a][r] = 0.f;
#pragma unroll
  for (int ks2 = 0; ks2 < 2 * WT; ++ks2) {
#pragma unroll
    for (int et = 0; et < ET; ++et) {
      const bf16x8 a = w2f[(int64_t)(ks2 * ET + et) * 64 + lane];
      acc2[et] = mfma_32x32x16<F16>(a, hb[ks2], acc2[et]);
    }
  }
  // norms (bf16 values held as float), per-token maximum
  float m = -INFINITY;
#pragma unroll
  for (int et = 0; et < ET; ++et)
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const uint32_t pk = enc16x2<F16>(fabsf(acc2[et][r]), fabsf(acc2[et][r + 1]));
      acc2[et][r] = dec16<F16>(pk & 0xffffu);
      acc2[et][r + 1] = dec16_hi<F16>(pk);
      m = nanmax(m, nanmax(acc2[et][r], acc2[et][r + 1]));
    }
  m = nanmax(m, __shfl_xor(m, 32, kWave));
  // (the product is rounded to float32 before it is rounded to the storage type: kept apart by the empty asm, or the
  // compiler folds multiply and float16 conversion into one instruction with a single rounding)
  float thr_prod = m * thr_scale;
  asm volatile("" : "+v"(thr_prod));
  const float thr = dec16<F16>(enc16x2<F16>(thr_prod, 0.f) & 0xffffu);
  // A lane holds 4 consecutive experts of one token per accumulator quad.  The rows go through a wave-private LDS tile
  // (16-byte pieces XORed with the row, so both directions spread over the banks) and leave as whole rows: CH lanes
  // write the E * 2 contiguous bytes of a token's routing (or norms) row.
  constexpr int CH = E / 8;            // 16-byte pieces per row
  constexpr int RPI = 64 / CH;         // rows per store instruction
  u32x4* stage = (u32x4*)stage_all + (threadIdx.x >> 6) * (32 * CH);
  const int srow = lane / CH, spc = lane % CH;
  auto flush = [&](bf16_t* dst) __attribute__((always_inline)) {
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
      const int row = srow + RPI * i;
      const u32x4 v = stage[row * CH + (spc ^ (row & (CH - 1)))];
      if (tok0 + row < N && spc * 8 < e_real) *(u32x4*)(dst + (tok0 + row) * e_real + spc * 8) = v;
    }
    __builtin_amdgcn_wave_barrier();
  };
  uint2* srow_w = (uint2*)(stage + c32 * CH);   // this lane's row; piece p at index (p ^ (c32 & (CH-1))) * 2 + g
  bool on[ET][16];
#pragma unroll
  for (int et = 0; et < ET; ++et) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int s = 0; s < 4; ++s) on[et][q * 4 + s] = acc2[et][q * 4 + s] >= thr;
      uint2 rv;
      rv.x = (on[et][q * 4 + 0] ? ONE : 0u) | (on[et][q * 4 + 1] ? (ONE << 16) : 0u);   // 1.0 in the storage type
      rv.y = (on[et][q * 4 + 2] ? ONE : 0u) | (on[et][q * 4 + 3] ? (ONE << 16) : 0u);
      srow_w[(((et * 4 + q) ^ (c32 & (CH - 1))) << 1) + g] = rv;
    }
  }
  flush(routing);
  if (norms_out != nullptr) {
#pragma unroll
    for (int et = 0; et < ET; ++et)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint2 nv;
        nv.x = enc16x2<F16>(acc2[et][q * 4 + 0], acc2[et][q * 4 + 1]);   // exact: the values are representable
        nv.y = enc16x2<F16>(acc2[et][q * 4 + 2], acc2[et][q * 4 + 3]);
        srow_w[(((et * 4 + q) ^ (c32 & (CH - 1))) << 1) + g] = nv;
      }
    flush(norms_out);
  }
  if (counts != nullptr) {
#pragma unroll
    for (int et = 0; et < ET; ++et)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const unsigned long long bal = __ballot(on[et][q * 4 + s] && valid);
          if (lane == 0 && et * 32 + 8 * q < e_real) {   // (experts come in blocks of 8: both indices are in or out)
            const int lo = __popcll(bal & 0xffffffffull), hi = __popcll(bal >> 32);
            if (lo) atomicAdd(counts + et * 32 + 8 * q + s, lo);
            if (hi) atomicAdd(counts + et * 32 + 8 * q + 4 + s, hi);
          }
        }
  }
}

// The same computation for launches that would leave most of the machine idle with one wave per 32 tokens (few tokens,
// long rows): a workgroup owns 32 tokens and its 4 waves share the OUTPUT features of each layer -- wave w computes
// hidden tiles [w*TW, (w+1)*TW) over all of K, the hidden activations are exchanged through LDS as B fragments, then
// wave w computes expert tiles [w*TE, (w+1)*TE); the per-token maximum is completed through LDS.  No partial sums are
// exchanged, so every value is bit-identical to the one-wave kernel's.  Loads run U K steps ahead in two register
// buffers.
typedef __attribute__((address_space(3))) void rs_lds_void;
template <int TW, int TE, int U, bool F16 = false, bool XL = false>
__global__ __launch_bounds__(256) void router_select_split_kernel(
    const bf16_t* __restrict__ x, const bf16x8* __restrict__ w1f, const bf16x8* __restrict__ w2f,
    bf16_t* __restrict__ routing, bf16_t* __restrict__ norms_out, int32_t* __restrict__ counts, int64_t N, int D,
    float thr_scale) {
  constexpr uint32_t ONE = F16 ? 0x3C00u : 0x3F80u;   // 1.0 in the storage type
  constexpr int WT = 4 * TW, ET = 4 * TE, E = ET * 32;
  __shared__ bf16x8 hs[2 * WT][64];
  __shared__ float smax[4][32];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = lane >> 5, c32 = lane & 31;
  const int64_t tok0 = (int64_t)blockIdx.x * 32;
  const int64_t token = tok0 + c32;
  const bool valid = token < N;
  const bf16x8* xrow = (const bf16x8*)(x + (valid ? token : (N - 1)) * D) + g;   // + 2 per K step
  const bf16x8* w1w = w1f + (int64_t)(w * TW) * 64 + lane;                       // + WT*64 per K step, + 64 per tile
  const int KS1 = D / 16;   // a multiple of 2*U (checked by the launcher)
  // XL: the x tile goes from global memory straight into LDS first (global_load_lds, 1 KB per wave instruction, 8 lanes
  // on 128 contiguous bytes of a row) and the B fragments are read from there: with long rows the four waves' fragment
  // reads straight from the rows (32 rows x 32 bytes per instruction, four times over) hold the kernel.  A 1 KB block
  // holds 8 pieces of 16 bytes of each of 8 rows; piece pp of row r of row group R sits at 16*(pp/2) + 2r + ((pp ^ R) & 1),
  // so the 16 tokens a quarter wave reads for one fragment fall into 16 different bank groups.
  extern __shared__ __attribute__((aligned(16))) unsigned char xl_raw[];
  const int XPR = D / 64;                               // blocks per row group
  const bf16x8* xl = (const bf16x8*)xl_raw + (c32 >> 3) * XPR * 64 + 2 * (c32 & 7) + ((g ^ (c32 >> 3)) & 1);
  if constexpr (XL) {
    const int dr = (lane >> 1) & 7, dpp = 2 * (lane >> 4) + ((lane ^ w) & 1);   // wave w moves row group w
    int64_t row = tok0 + 8 * w + dr;
    row = row < N ? row : N - 1;
    const bf16_t* src = x + row * D + dpp * 8;
    unsigned char* dst = xl_raw + (size_t)w * XPR * 1024;
    for (int j = 0; j < XPR; ++j) __builtin_amdgcn_global_load_lds(src + j * 64, (rs_lds_void*)(dst + j * 1024), 16, 0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
  }

  f32x16 acc1[TW];
#pragma unroll
  for (int a = 0; a < TW; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[a][r] = 0.f;
  bf16x8 xA[U], wA[U][TW], xB[U], wB[U][TW];
  auto fill = [&](bf16x8 (&xb)[U], bf16x8 (&wr)[U][TW], int ks0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if constexpr (XL) xb[u] = xl[((ks0 + u) >> 2) * 64 + ((ks0 + u) & 3) * 16];
      else xb[u] = xrow[2 * (ks0 + u)];
#pragma unroll
      for (int a = 0; a < TW; ++a) wr[u][a] = w1w[((int64_t)(ks0 + u) * WT + a) * 64];
    }
  };
  auto multiply = [&](bf16x8 (&xb)[U], bf16x8 (&wr)[U][TW]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int a = 0; a < TW; ++a) acc1[a] = mfma_32x32x16<F16>(wr[u][a], xb[u], acc1[a]);
  };
  fill(xA, wA, 0);
  for (int ks0 = 0; ks0 < KS1; ks0 += 2 * U) {
    fill(xB, wB, ks0 + U);
    multiply(xA, wA);
    fill(xA, wA, (ks0 + 2 * U < KS1) ? (ks0 + 2 * U) : ks0);   // the last trip re-reads its own steps: in bounds, unused
    multiply(xB, wB);
  }
  // the first TE expert-tile fragments of the second layer are requested before the exchange
  const bf16x8* w2w = w2f + (int64_t)(w * TE) * 64 + lane;   // + ET*64 per K step, + 64 per tile
  // hidden activations -> LDS as B fragments of the second product
#pragma unroll
  for (int a = 0; a < TW; ++a)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint4 pk;
      pk.x = enc16x2<F16>(fmaxf(acc1[a][half * 8 + 0], 0.f), fmaxf(acc1[a][half * 8 + 1], 0.f));
      pk.y = enc16x2<F16>(fmaxf(acc1[a][half * 8 + 2], 0.f), fmaxf(acc1[a][half * 8 + 3], 0.f));
      pk.z = enc16x2<F16>(fmaxf(acc1[a][half * 8 + 4], 0.f), fmaxf(acc1[a][half * 8 + 5], 0.f));
      pk.w = enc16x2<F16>(fmaxf(acc1[a][half * 8 + 6], 0.f), fmaxf(acc1[a][half * 8 + 7], 0.f));
      ((uint4*)hs)[((w * TW + a) * 2 + half) * 64 + lane] = pk;
    }
  __syncthreads();
  f32x16 acc2[TE];
#pragma unroll
  for (int a = 0; a < TE; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc2[a][r] = 0.f;
  for (int k0 = 0; k0 < 2 * WT; k0 += 8) {   // 2*WT is a multiple of 8
    bf16x8 a2[8][TE];
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
      for (int et = 0; et < TE; ++et) a2[k][et] = w2w[((int64_t)(k0 + k) * ET + et) * 64];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const bf16x8 hb = hs[k0 + k][lane];
#pragma unroll
      for (int et = 0; et < TE; ++et) acc2[et] = mfma_32x32x16<F16>(a2[k][et], hb, acc2[et]);
    }
  }
  // norms (bf16 values held as float), per-token maximum over this wave's experts, then over the four waves
  float m = -INFINITY;
#pragma unroll
  for (int et = 0; et < TE; ++et)
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const uint32_t pk = enc16x2<F16>(fabsf(acc2[et][r]), fabsf(acc2[et][r + 1]));
      acc2[et][r] = dec16<F16>(pk & 0xffffu);
      acc2[et][r + 1] = dec16_hi<F16>(pk);
      m = nanmax(m, nanmax(acc2[et][r], acc2[et][r + 1]));
    }
  m = nanmax(m, __shfl_xor(m, 32, kWave));
  if (g == 0) smax[w][c32] = m;
  __syncthreads();
  m = nanmax(nanmax(smax[0][c32], smax[1][c32]), nanmax(smax[2][c32], smax[3][c32]));
  // (the product is rounded to float32 before it is rounded to the storage type: kept apart by the empty asm, or the
  // compiler folds multiply and float16 conversion into one instruction with a single rounding)
  float thr_prod = m * thr_scale;
  asm volatile("" : "+v"(thr_prod));
  const float thr = dec16<F16>(enc16x2<F16>(thr_prod, 0.f) & 0xffffu);
#pragma unroll
  for (int et = 0; et < TE; ++et) {
    const int etg = w * TE + et;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e0 = etg * 32 + 8 * q + 4 * g;
      bool on[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) on[s] = acc2[et][q * 4 + s] >= thr;
      if (valid) {
        uint2 rv;
        rv.x = (on[0] ? ONE : 0u) | (on[1] ? (ONE << 16) : 0u);   // 1.0 in the storage type
        rv.y = (on[2] ? ONE : 0u) | (on[3] ? (ONE << 16) : 0u);
        *(uint2*)(routing + token * E + e0) = rv;
        if (norms_out != nullptr) {
          uint2 nv;
          nv.x = enc16x2<F16>(acc2[et][q * 4 + 0], acc2[et][q * 4 + 1]);   // exact: the values are representable
          nv.y = enc16x2<F16>(acc2[et][q * 4 + 2], acc2[et][q * 4 + 3]);
          *(uint2*)(norms_out + token * E + e0) = nv;
        }
      }
      if (counts != nullptr) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const unsigned long long bal = __ballot(on[s] && valid);
          if (lane == 0) {
            const int lo = __popcll(bal & 0xffffffffull), hi = __popcll(bal >> 32);
            if (lo) atomicAdd(counts + etg * 32 + 8 * q + s, lo);
            if (hi) atomicAdd(counts + etg * 32 + 8 * q + 4 + s, hi);
          }
        }
      }
    }
  }
}

// The same computation for many tokens of a router whose first layer fits the register file (D = 768, width 128:
// 192 registers per lane): one workgroup per CU walks the tiles of 32 tokens, wave w keeps the A fragments of hidden
// tile w (all of K) and of expert tile w in registers for the whole launch, so the only stream through the CU is x itself
// (the kernels above fetch the 196 KB of first-layer fragments from L2 for every 32 tokens, four times the bytes of x).
// The x tiles go from global memory straight into LDS (global_load_lds: a wave instruction moves 64 x 16 bytes to 1 KB
// of consecutive LDS, whatever the lanes' global addresses), two tiles ahead of the one being multiplied, into three
// buffers.  A 1 KB block holds 128 bytes (8 pieces of 16) of each of 8 rows; piece pp of row r of row group R sits at
// position 16*(pp/2) + 2r + ((pp ^ R) & 1): two neighbouring lanes fetch 32 contiguous bytes, and the 16 tokens a quarter
// wave reads for one B fragment (same piece, rows of two row groups) fall into 16 different 16-byte bank groups.
// Hidden activations, row maxima and the routing / norms rows are exchanged through LDS as in the split kernel (the
// rows where the hidden activations were); every accumulator chain runs over K in
// ascending order, so all three kernels give the same bits.  Per-expert counts are kept in registers over the tiles
// and added once per wave.
typedef __attribute__((address_space(3))) void rr_lds_void;
constexpr int RR_D = 768;
constexpr int RR_TILE_BYTES = 32 * RR_D * 2;
constexpr size_t RR_LDS = (size_t)3 * RR_TILE_BYTES + 8 * 64 * 16 + 4 * 32 * sizeof(float) + 4 * sizeof(int);

template <int D, bool F16 = false>
__global__ __launch_bounds__(256, 1) void router_select_resident_kernel(
    const bf16_t* __restrict__ x, const bf16x8* __restrict__ w1f, const bf16x8* __restrict__ w2f,
    bf16_t* __restrict__ routing, bf16_t* __restrict__ norms_out, int32_t* __restrict__ counts,
    int32_t* __restrict__ seg_counts, int32_t* __restrict__ seg_pairs, int64_t N, float thr_scale) {
  constexpr uint32_t ONE = F16 ? 0x3C00u : 0x3F80u;   // 1.0 in the storage type
  constexpr int KS1 = D / 16, E = 128, CH = 16;
  constexpr int XP = KS1 / 4;                          // 1 KB blocks per wave and tile (groups of 8 pieces per row)
  constexpr int TB = RR_TILE_BYTES / 16;               // tile buffer in 16-byte units
  static_assert(D == RR_D, "the LDS budget is written for D = 768");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* xs = (u32x4*)smem_raw;                        // [3][4 row groups][XP blocks][64]
  u32x4* hs = xs + 3 * TB;                             // [8][64]
  float* smax = (float*)(hs + 8 * 64);                 // [4][32]
  int* spair = (int*)(smax + 4 * 32);                  // [4]: the waves' routed pairs of the tile
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = lane >> 5, c32 = lane & 31;
  const int64_t n_tiles = (N + 31) / 32;
  const int64_t G = gridDim.x;
  const bool counting = counts != nullptr || seg_counts != nullptr;   // uniform

  // x rows -> LDS: wave w moves row group w (rows 8w .. 8w+7); lane = 16a + 2r + par fetches piece 2a + (par ^ (w & 1))
  // of the block's 8, of row r
  const int dr = (lane >> 1) & 7, dpp = 2 * (lane >> 4) + ((lane ^ w) & 1);
  auto issue_part = [&](int64_t t, int buf, int j0, int j1) __attribute__((always_inline)) {
    int64_t row = t * 32 + 8 * w + dr;
    row = row < N ? row : N - 1;                       // rows past the end: the last row again (unused)
    const bf16_t* src = x + row * D + dpp * 8;
    unsigned char* dst = smem_raw + (size_t)buf * RR_TILE_BYTES + (size_t)w * XP * 1024;
#pragma unroll
    for (int j = j0; j < j1; ++j)
      __builtin_amdgcn_global_load_lds(src + j * 64, (rr_lds_void*)(dst + j * 1024), 16, 0, 0);
  };
  auto issue = [&](int64_t t, int buf) __attribute__((always_inline)) { issue_part(t, buf, 0, XP); };
  int64_t tile = blockIdx.x;
  issue(tile, 0);
  issue(tile + G < n_tiles ? tile + G : tile, 1);

  bf16x8 w1r[KS1], w2r[8];
#pragma unroll
  for (int ks = 0; ks < KS1; ++ks) w1r[ks] = w1f[(int64_t)(ks * 4 + w) * 64 + lane];
#pragma unroll
  for (int k = 0; k < 8; ++k) w2r[k] = w2f[(int64_t)(k * 4 + w) * 64 + lane];
  // the weights are waited for here, once: left pending into the loop, every trip would wait for them again
#pragma unroll
  for (int ks = 0; ks < KS1; ++ks) asm volatile("" : "+v"(w1r[ks]));
#pragma unroll
  for (int k = 0; k < 8; ++k) asm volatile("" : "+v"(w2r[k]));
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // ... and with them the first two tiles

  // B fragment of K step ks, half g, token c32 = row c32 % 8 of row group c32 / 8: block ks / 4 of the group, position
  // 16*(ks % 4) + 2r + ((g ^ R) & 1)
  const int xrd = (c32 >> 3) * XP * 64 + 2 * (c32 & 7) + ((g ^ (c32 >> 3)) & 1);
  int cnt = 0;                                         // lanes 0..31: tokens routed to expert 32w + lane so far
  const int frow = threadIdx.x >> 4, fpc = threadIdx.x & 15;   // flush: 16 lanes write one 256-byte row

  for (int it = 0; tile < n_tiles; tile += G, ++it) {
    const int buf = it % 3;
    const int64_t tok0 = tile * 32;
    const bool valid = tok0 + c32 < N;
    lds_barrier();                                     // every wave's pieces of this tile have landed (it waited for its
                                                       // own below), and the buffer of the tile before is free
    // the tile after next is requested two blocks at a time between the groups of products below (all twelve at once
    // keep the wave at the issue of its loads for longer than the first products take)
    const int64_t ahead = tile + 2 * G < n_tiles ? tile + 2 * G : tile;   // past the end: this tile's rows again, unused
    constexpr int XI = XP / (KS1 / 8);                 // blocks per group of 8 K steps
    static_assert(XI * (KS1 / 8) == XP, "the requests are dealt evenly over the groups of products");
    f32x16 acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[r] = 0.f;
    // fragments are read a group of XG K steps ahead of the products that use them (two register groups)
    constexpr int XG = 8;
    static_assert(KS1 % (2 * XG) == 0, "K steps come in pairs of groups");
    u32x4 fa[XG], fb[XG];
    const u32x4* xt = xs + buf * TB + xrd;
    auto fetch = [&](u32x4 (&f)[XG], int ks0) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < XG; ++u) f[u] = xt[((ks0 + u) >> 2) * 64 + ((ks0 + u) & 3) * 16];
    };
    auto product = [&](u32x4 (&f)[XG], int ks0) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < XG; ++u) {
        bf16x8 b;
        __builtin_memcpy(&b, &f[u], 16);
        acc1 = mfma_32x32x16<F16>(w1r[ks0 + u], b, acc1);
      }
    };
    fetch(fa, 0);
#pragma unroll
    for (int ks0 = 0; ks0 < KS1; ks0 += 2 * XG) {
      fetch(fb, ks0 + XG);
      __builtin_amdgcn_sched_barrier(0);
      product(fa, ks0);
      __builtin_amdgcn_sched_barrier(0);
      issue_part(ahead, (it + 2) % 3, (ks0 / XG) * XI, (ks0 / XG + 1) * XI);
      __builtin_amdgcn_sched_barrier(0);
      if (ks0 + 2 * XG < KS1) fetch(fa, ks0 + 2 * XG);
      __builtin_amdgcn_sched_barrier(0);
      product(fb, ks0 + XG);
      __builtin_amdgcn_sched_barrier(0);
      issue_part(ahead, (it + 2) % 3, (ks0 / XG + 1) * XI, (ks0 / XG + 2) * XI);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      u32x4 pk;
      pk.x = enc16x2<F16>(fmaxf(acc1[half * 8 + 0], 0.f), fmaxf(acc1[half * 8 + 1], 0.f));
      pk.y = enc16x2<F16>(fmaxf(acc1[half * 8 + 2], 0.f), fmaxf(acc1[half * 8 + 3], 0.f));
      pk.z = enc16x2<F16>(fmaxf(acc1[half * 8 + 4], 0.f), fmaxf(acc1[half * 8 + 5], 0.f));
      pk.w = enc16x2<F16>(fmaxf(acc1[half * 8 + 6], 0.f), fmaxf(acc1[half * 8 + 7], 0.f));
      hs[(w * 2 + half) * 64 + lane] = pk;
    }
    lds_barrier();                                     // from here on nobody reads this tile's x buffer
    f32x16 acc2;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc2[r] = 0.f;
    u32x4 hv[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) hv[k] = hs[k * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      bf16x8 hb;
      __builtin_memcpy(&hb, &hv[k], 16);
      acc2 = mfma_32x32x16<F16>(w2r[k], hb, acc2);
    }
    // norms (storage-type values held as float), per-token maximum over this wave's experts, then over the four waves
    float m = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const uint32_t pk = enc16x2<F16>(fabsf(acc2[r]), fabsf(acc2[r + 1]));
      acc2[r] = dec16<F16>(pk & 0xffffu);
      acc2[r + 1] = dec16_hi<F16>(pk);
      m = nanmax(m, nanmax(acc2[r], acc2[r + 1]));
    }
    m = nanmax(m, __shfl_xor(m, 32, kWave));
    if (g == 0) smax[w * 32 + c32] = m;
    lds_barrier();
    m = nanmax(nanmax(smax[c32], smax[32 + c32]), nanmax(smax[64 + c32], smax[96 + c32]));
    // (the product is rounded to float32 before it is rounded to the storage type: kept apart by the empty asm, or the
    // compiler folds multiply and float16 conversion into one instruction with a single rounding)
    float thr_prod = m * thr_scale;
    asm volatile("" : "+v"(thr_prod));
    const float thr = dec16<F16>(enc16x2<F16>(thr_prod, 0.f) & 0xffffu);
    // routing rows (then norms rows): 32 rows of 16 pieces each, where the hidden activations were
    // (written with ds_write_b64 spelled out: before an ordinary LDS store the compiler waits for every global_load_lds
    // in flight, the tile after next included; the barriers below wait for these writes like for any other)
    const uint32_t srow = (uint32_t)(uintptr_t)(rr_lds_void*)(hs + c32 * CH);   // this lane's row; piece p, half g at
    auto put = [&](int piece, const uint2& v) __attribute__((always_inline)) {  // byte ((p ^ (c32 & 15)) * 2 + g) * 8
      asm volatile("ds_write_b64 %0, %1" :: "v"(srow + (uint32_t)((((piece ^ (c32 & (CH - 1))) << 1) + g) << 3)), "v"(v) : "memory");
    };
    int tcnt = 0;                                      // lanes 0..31: this tile's tokens routed to expert 32w + lane
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      bool on[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) on[s] = acc2[q * 4 + s] >= thr;
      uint2 rv;
      rv.x = (on[0] ? ONE : 0u) | (on[1] ? (ONE << 16) : 0u);
      rv.y = (on[2] ? ONE : 0u) | (on[3] ? (ONE << 16) : 0u);
      put(w * 4 + q, rv);
      if (counting) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const unsigned long long bal = __ballot(on[s] && valid);   // low half: expert 8q + s, high half: 8q + 4 + s
          tcnt = (lane == 8 * q + s) ? __popcll(bal & 0xffffffffull) : tcnt;
          tcnt = (lane == 8 * q + 4 + s) ? __popcll(bal >> 32) : tcnt;
        }
      }
    }
    cnt += tcnt;
    if (seg_counts != nullptr) {
      // the expert-major plan's first pass, for the segment of 32 tokens this tile is: tokens per expert, pairs in all
      if (lane < 32) seg_counts[tile * E + w * 32 + lane] = tcnt;
      const int wp = wave_sum_i32(tcnt);
      if (lane == 0) spair[w] = wp;
    }
    lds_barrier();
    if (seg_counts != nullptr && threadIdx.x == 0) seg_pairs[tile] = spair[0] + spair[1] + spair[2] + spair[3];
    // This wave's pieces of the NEXT tile have landed once only the XP loads issued in this trip are still in flight
    // (the stores below come after the wait, the ones of the trip before are older than those loads).
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(XP) : "memory");
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = frow + 16 * i;
      if (tok0 + row < N) *(u32x4*)(routing + (tok0 + row) * E + fpc * 8) = hs[row * CH + (fpc ^ (row & (CH - 1)))];
    }
    if (norms_out != nullptr) {                        // uniform
      lds_barrier();
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint2 nv;
        nv.x = enc16x2<F16>(acc2[q * 4 + 0], acc2[q * 4 + 1]);   // exact: the values are representable
        nv.y = enc16x2<F16>(acc2[q * 4 + 2], acc2[q * 4 + 3]);
        put(w * 4 + q, nv);
      }
      lds_barrier();
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = frow + 16 * i;
        if (tok0 + row < N) *(u32x4*)(norms_out + (tok0 + row) * E + fpc * 8) = hs[row * CH + (fpc ^ (row & (CH - 1)))];
      }
    }
  }
  if (counts != nullptr && lane < 32 && cnt != 0) atomicAdd(counts + w * 32 + lane, cnt);
}

// Per-expert token counts of a routing mask [N, E] in 16-bit storage, E = 64 * EPL: column sums of the non-zero entries.
// Behind the split kernel, whose workgroups own 32 tokens each: one integer atomic per expert and workgroup from a few
// hundred workgroups queues up on the four cache lines of the counters (8192 tokens: 16 -> 95 us); here a workgroup
// takes a long run of rows, lanes = experts, and adds once.
template <int EPL>
__global__ __launch_bounds__(256) void routing_counts_kernel(const bf16_t* __restrict__ routing, int32_t* __restrict__ counts,
                                                             int64_t N, int64_t rows_per_wg) {
  constexpr int E = 64 * EPL;
  typedef uint16_t row_piece __attribute__((ext_vector_type(EPL)));
  __shared__ int part[4][E];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_wg;
  const int64_t r1 = (r0 + rows_per_wg < N) ? (r0 + rows_per_wg) : N;
  int cnt[EPL];
#pragma unroll
  for (int k = 0; k < EPL; ++k) cnt[k] = 0;
  constexpr int UN = 8;
  for (int64_t r = r0 + w; r < r1; r += 4 * UN) {
    row_piece v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int64_t rr = (r + 4 * u < r1) ? (r + 4 * u) : (r1 - 1);   // clamped: the loads go out together
      v[u] = *(const row_piece*)(routing + rr * E + lane * EPL);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int k = 0; k < EPL; ++k) cnt[k] += (r + 4 * u < r1 && (v[u][k] & 0x7fff) != 0) ? 1 : 0;
  }
#pragma unroll
  for (int k = 0; k < EPL; ++k) part[w][lane * EPL + k] = cnt[k];
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 256) {
    const int t = part[0][e] + part[1][e] + part[2][e] + part[3][e];
    if (t != 0) atomicAdd(counts + e, t);
  }
}

bool mfma_router_writes_plan_counts(const d2dmoe_shape& sh) {
  return mfma_router_supported(sh) && router_shape_exact(sh) && sh.d_model == RR_D && sh.router_width == 128 &&
         sh.n_tokens >= (int64_t)64 * device_cu_count();
}

template <bool F16>
static hipError_t launch_mfma_router_select_t(const d2dmoe_shape& sh, const void* x, const void* packed, void* routing,
                                     void* norms_out, int32_t* counts, float thr_scale, int32_t* seg_counts,
                                     int32_t* seg_pairs, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  if (!L.has_router) return hipErrorInvalidValue;
  const char* base = (const char*)packed;
  if (counts != nullptr) {
    hipError_t e = launch_fill_i32(counts, sh.n_experts, 0, s);
    if (e != hipSuccess) return e;
  }
  const bf16_t* xp = (const bf16_t*)x;
  const bf16x8* r1 = (const bf16x8*)(base + L.r1_off);
  const bf16x8* r2 = (const bf16x8*)(base + L.r2_off);
  // One wave per 32 tokens fills the machine from about 4 * 32 * CUs tokens on; below that (or with long rows, where a
  // wave's K loop is the critical path) a workgroup per 32 tokens shares the output features among its waves.
  const int cus = device_cu_count();
  if (mfma_router_writes_plan_counts(sh)) {
    auto kern = router_select_resident_kernel<RR_D, F16>;
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RR_LDS);
    if (e != hipSuccess) return e;
    const int64_t n_tiles = cdiv64(sh.n_tokens, 32);
    hipLaunchKernelGGL(kern, dim3((unsigned)(n_tiles < cus ? n_tiles : cus)), dim3(256), RR_LDS, s, xp, r1, r2, (bf16_t*)routing,
                       (bf16_t*)norms_out, counts, seg_counts, seg_pairs, sh.n_tokens, thr_scale);
    return hipGetLastError();
  }
  const bool split = router_shape_exact(sh) && (sh.n_tokens < (int64_t)128 * cus || sh.d_model >= 2048) && (sh.d_model / 16) % 4 == 0;
  if (split) {
    const unsigned grid = (unsigned)cdiv64(sh.n_tokens, 32);
    const bool deep = (sh.d_model / 16) % 8 == 0;
    // from a few hundred workgroups on, the counts are taken from the finished mask by a kernel of their own
    const bool count_after = counts != nullptr && grid > 64;
    int32_t* kc = count_after ? nullptr : counts;
    if (sh.router_width == 128) {
      if (deep) hipLaunchKernelGGL((router_select_split_kernel<1, 1, 4, F16>), dim3(grid), dim3(256), 0, s, xp, r1, r2, (bf16_t*)routing,
                                   (bf16_t*)norms_out, kc, sh.n_tokens, sh.d_model, thr_scale);
      else hipLaunchKernelGGL((router_select_split_kernel<1, 1, 2, F16>), dim3(grid), dim3(256), 0, s, xp, r1, r2, (bf16_t*)routing,
                              (bf16_t*)norms_out, kc, sh.n_tokens, sh.d_model, thr_scale);
    } else {
      // long rows (the Gemma router: 2048 -> 256 -> 256): the x tile is staged in LDS (128 KB at D = 2048, the most that
      // fits beside the exchanged activations): 26.7 -> 16.3 us at 1030 tokens, 29 -> 22 us at 4096
      if (deep && sh.d_model >= 1536 && sh.d_model <= 2048) {
        auto kern = router_select_split_kernel<2, 2, 4, F16, true>;
        const size_t xl_bytes = (size_t)32 * sh.d_model * 2;
        hipError_t e2 = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)xl_bytes);
        if (e2 != hipSuccess) return e2;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), xl_bytes, s, xp, r1, r2, (bf16_t*)routing,
                           (bf16_t*)norms_out, kc, sh.n_tokens, sh.d_model, thr_scale);
      } else if (deep) hipLaunchKernelGGL((router_select_split_kernel<2, 2, 4, F16>), dim3(grid), dim3(256), 0, s, xp, r1, r2, (bf16_t*)routing,
                                   (bf16_t*)norms_out, kc, sh.n_tokens, sh.d_model, thr_scale);
      else hipLaunchKernelGGL((router_select_split_kernel<2, 2, 2, F16>), dim3(grid), dim3(256), 0, s, xp, r1, r2, (bf16_t*)routing,
                              (bf16_t*)norms_out, kc, sh.n_tokens, sh.d_model, thr_scale);
    }
    if (count_after) {
      const int64_t rows_per_wg = cdiv64(sh.n_tokens, 32);   // 32 workgroups
      const unsigned cgrid = (unsigned)cdiv64(sh.n_tokens, rows_per_wg);
      if (sh.n_experts == 128)
        hipLaunchKernelGGL(routing_counts_kernel<2>, dim3(cgrid), dim3(256), 0, s, (const bf16_t*)routing, counts, sh.n_tokens, rows_per_wg);
      else
        hipLaunchKernelGGL(routing_counts_kernel<4>, dim3(cgrid), dim3(256), 0, s, (const bf16_t*)routing, counts, sh.n_tokens, rows_per_wg);
    }
    return hipGetLastError();
  }
  const unsigned grid = (unsigned)cdiv64(sh.n_tokens, 128);
  const bool deep = (sh.d_model / 16) % 8 == 0;
#define D2DMOE_ROUTER(WT, ET, U)                                                                                         \
  hipLaunchKernelGGL((router_select_mfma_kernel<WT, ET, U, F16>), dim3(grid), dim3(256), 0, s, xp, r1, r2, (bf16_t*)routing, \
                     (bf16_t*)norms_out, counts, sh.n_tokens, sh.d_model, thr_scale, sh.n_experts)
  if (sh.router_width == 128) {
    switch (mfma_router_padded_experts(sh)) {
      case 32: if (deep) D2DMOE_ROUTER(4, 1, 4); else D2DMOE_ROUTER(4, 1, 2); break;
      case 64: if (deep) D2DMOE_ROUTER(4, 2, 4); else D2DMOE_ROUTER(4, 2, 2); break;
      case 128: if (deep) D2DMOE_ROUTER(4, 4, 4); else D2DMOE_ROUTER(4, 4, 2); break;
      default: if (deep) D2DMOE_ROUTER(4, 8, 4); else D2DMOE_ROUTER(4, 8, 2); break;
    }
  } else {
    D2DMOE_ROUTER(8, 8, 2);
  }
#undef D2DMOE_ROUTER
  return hipGetLastError();
}

// seg_counts / seg_pairs (optional): the expert-major plan's per-segment counts, written by the kernel when
// mfma_router_writes_plan_counts(sh) holds and ignored otherwise.
hipError_t launch_mfma_router_select(const d2dmoe_shape& sh, const void* x, const void* packed, void* routing,
                                     void* norms_out, int32_t* counts, float thr_scale, hipStream_t s, int32_t* seg_counts,
                                     int32_t* seg_pairs) {
  if (sh.dtype == D2DMOE_F16)
    return launch_mfma_router_select_t<true>(sh, x, packed, routing, norms_out, counts, thr_scale, seg_counts, seg_pairs, s);
  return launch_mfma_router_select_t<false>(sh, x, packed, routing, norms_out, counts, thr_scale, seg_counts, seg_pairs, s);
}

}  // namespace d2dmoe
