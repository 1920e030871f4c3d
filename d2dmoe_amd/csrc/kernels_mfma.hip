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
#include "common.hpp"
#include "launch.hpp"

namespace d2dmoe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int MD_BM = 64;       // tokens per workgroup
constexpr int MD_HC = 256;      // hidden neurons per chunk (4 waves x 64)
constexpr int MD_WAVES = 4;
constexpr int MD_KS2 = MD_HC / 16;  // K=16 steps of the second GEMM per chunk

struct PackedLayout {
  int hidden;      // E * Ed
  int n_chunks;    // ceil(hidden / MD_HC)
  int hidden_pad;  // n_chunks * MD_HC
  size_t w1_off, w2_off, b1_off, eidx_off, total;
};

static PackedLayout packed_layout(const d2dmoe_shape& sh) {
  PackedLayout L;
  L.hidden = sh.n_experts * sh.expert_dim;
  L.n_chunks = (L.hidden + MD_HC - 1) / MD_HC;
  L.hidden_pad = L.n_chunks * MD_HC;
  size_t off = 0;
  L.w1_off = off;   off += (size_t)L.hidden_pad * sh.d_model * 2;
  L.w2_off = off;   off += (size_t)L.hidden_pad * sh.d_model * 2;
  L.b1_off = off;   off += (size_t)L.hidden_pad * 4;
  L.eidx_off = off; off += (size_t)L.hidden_pad * 2;
  L.total = (off + 255) / 256 * 256;
  return L;
}

bool mfma_dense_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 || sh.gated) return false;
  if (sh.d_model != 768) return false;
  if (sh.n_experts > 128) return false;          // routing tile [64][E] bf16 must fit beside the x and h tiles
  const int hidden = sh.n_experts * sh.expert_dim;
  if ((hidden + MD_HC - 1) / MD_HC > 64) return false;
  return true;
}

size_t mfma_packed_bytes(const d2dmoe_shape& sh) { return packed_layout(sh).total; }

// ---------------------------------------------------------------------------------------------------
// Packing.  One thread per 16-byte fragment piece.
//   W1 fragments  [chunk][wave][kstep D/16][row-tile 2][lane 64][8]:
//       neuron h = chunk*256 + wave*64 + rt*32 + c,  d = kstep*16 + 8g + i        value w1[h/Ed][d][h%Ed]
//   W2 fragments  [chunk][wave][kstep2 16][col-tile D/128][lane 64][8]:
//       neuron h = chunk*256 + (ks2/2)*32 + (ks2%2)*16 + 8*(i/4) + 4g + (i%4)
//       column   = wave*(D/4) + ct*32 + c                                         value w2[h/Ed][h%Ed][column]
//   b1 as float [hidden_pad], expert index of every neuron as uint16 [hidden_pad]; padding neurons are zero.
// ---------------------------------------------------------------------------------------------------
__global__ void pack_w1_kernel(const bf16_t* __restrict__ w1, bf16_t* __restrict__ dst, int D, int Ed, int hidden,
                               int64_t n_pieces) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_pieces) return;
  const int KS1 = D / 16;
  const int lane = (int)(p % 64);
  int64_t q = p / 64;
  const int rt = (int)(q % 2); q /= 2;
  const int ks = (int)(q % KS1); q /= KS1;
  const int wave = (int)(q % MD_WAVES);
  const int chunk = (int)(q / MD_WAVES);
  const int g = lane / 32, c = lane % 32;
  const int h = chunk * MD_HC + wave * 64 + rt * 32 + c;
  bf16_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = ks * 16 + 8 * g + i;
    v[i] = (h < hidden) ? w1[((int64_t)(h / Ed) * D + d) * Ed + (h % Ed)] : (bf16_t)0;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) dst[p * 8 + i] = v[i];
}

__global__ void pack_w2_kernel(const bf16_t* __restrict__ w2, bf16_t* __restrict__ dst, int D, int Ed, int hidden,
                               int64_t n_pieces) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_pieces) return;
  const int CT = D / 128;
  const int lane = (int)(p % 64);
  int64_t q = p / 64;
  const int ct = (int)(q % CT); q /= CT;
  const int ks2 = (int)(q % MD_KS2); q /= MD_KS2;
  const int wave = (int)(q % MD_WAVES);
  const int chunk = (int)(q / MD_WAVES);
  const int g = lane / 32, c = lane % 32;
  const int col = wave * (D / 4) + ct * 32 + c;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int h = chunk * MD_HC + (ks2 / 2) * 32 + (ks2 % 2) * 16 + 8 * (i / 4) + 4 * g + (i % 4);
    dst[p * 8 + i] = (h < hidden) ? w2[((int64_t)(h / Ed) * Ed + (h % Ed)) * D + col] : (bf16_t)0;
  }
}

__global__ void pack_bias_kernel(const bf16_t* __restrict__ b1, float* __restrict__ b1p, uint16_t* __restrict__ eidx,
                                 int Ed, int hidden, int hidden_pad) {
  const int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= hidden_pad) return;
  b1p[h] = (h < hidden && b1 != nullptr) ? bf16_to_f32(b1[h]) : 0.f;
  eidx[h] = (uint16_t)((h < hidden) ? (h / Ed) : 0);
}

hipError_t launch_mfma_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            const void* router_w1, const void* router_w2, void* packed, hipStream_t s) {
  (void)w_up; (void)router_w1; (void)router_w2;
  const PackedLayout L = packed_layout(sh);
  char* base = (char*)packed;
  const int64_t n_pieces = (int64_t)L.hidden_pad * sh.d_model / 8;
  const unsigned blocks = (unsigned)((n_pieces + 255) / 256);
  hipLaunchKernelGGL(pack_w1_kernel, dim3(blocks), dim3(256), 0, s, (const bf16_t*)w1, (bf16_t*)(base + L.w1_off),
                     sh.d_model, sh.expert_dim, L.hidden, n_pieces);
  hipLaunchKernelGGL(pack_w2_kernel, dim3(blocks), dim3(256), 0, s, (const bf16_t*)w2, (bf16_t*)(base + L.w2_off),
                     sh.d_model, sh.expert_dim, L.hidden, n_pieces);
  hipLaunchKernelGGL(pack_bias_kernel, dim3((L.hidden_pad + 255) / 256), dim3(256), 0, s, (const bf16_t*)b1,
                     (float*)(base + L.b1_off), (uint16_t*)(base + L.eidx_off), sh.expert_dim, L.hidden, L.hidden_pad);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Fused experts kernel, token-tile-major ("masked dense sweep").
// Workgroup = 4 waves, 64 tokens.  LDS: the x tile as B fragments (96 KB at D = 768, resident for the whole
// kernel), one chunk of h as A fragments (32 KB), the routing tile (64 x E bf16).  Per chunk of 256 neurons:
//   GEMM1  wave w: H^T[64 neurons of w, 64 tokens] over K = D        A = W1 fragments (global), B = x (LDS)
//   epilogue      + b1, activation, round to bf16, x routing[token, expert(neuron)], store as A fragments to LDS
//   GEMM2  wave w: OUT[64 tokens, D/4 columns of w] += H . W2         A = h (LDS), B = W2 fragments (global)
// OUT stays in registers across all chunks (ascending neuron = ascending expert order, float32) and is rounded
// once in the final epilogue (+ last_bias, + x).  Chunks none of whose experts is routed to by any token of the
// tile are skipped (uniform branch).
// ---------------------------------------------------------------------------------------------------
__device__ inline uint32_t pack2_bf16(float lo, float hi) {
  return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}

template <int D, int ACT>
__global__ __launch_bounds__(256, 1) void experts_mfma_dense_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ routing, const bf16x8* __restrict__ w1p,
    const bf16x8* __restrict__ w2p, const float* __restrict__ b1p, const uint16_t* __restrict__ eidx,
    const bf16_t* __restrict__ last_bias, bf16_t* __restrict__ out, int64_t N, int E, int n_chunks, int hidden,
    int act_rt, int add_residual) {
  constexpr int KS1 = D / 16;   // K steps of GEMM1
  constexpr int CT = D / 128;   // 32-wide column tiles per wave in GEMM2
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16x8* xs = (bf16x8*)smem_raw;                              // [2][KS1][64]
  bf16x8* hs = xs + 2 * KS1 * 64;                              // [2][MD_KS2][64]
  bf16_t* rs = (bf16_t*)(hs + 2 * MD_KS2 * 64);                // [64][E]
  int* eact = (int*)(rs + MD_BM * E);                          // [E] then chunk flags [n_chunks]
  int* cact = eact + E;

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int w = t >> 6;
  const int g = lane >> 5, c32 = lane & 31;
  const int64_t tok0 = (int64_t)blockIdx.x * MD_BM;

  // ---- stage x (as B fragments) and routing
  {
    constexpr int PIECES_PER_ROW = D / 8;
    const uint4 zero4 = {0u, 0u, 0u, 0u};
    for (int p = t; p < MD_BM * PIECES_PER_ROW; p += 256) {
      const int m = p / PIECES_PER_ROW, kk = p - m * PIECES_PER_ROW;
      const int64_t n = tok0 + m;
      uint4 v = (n < N) ? *(const uint4*)(x + n * D + kk * 8) : zero4;
      const int ks = kk >> 1, gg = kk & 1;
      ((uint4*)xs)[((m >> 5) * KS1 + ks) * 64 + (m & 31) + 32 * gg] = v;
    }
    for (int i = t; i < MD_BM * E; i += 256) {
      const int m = i / E;
      const int64_t n = tok0 + m;
      rs[i] = (n < N) ? routing[n * E + (i - m * E)] : (bf16_t)0;
    }
    for (int i = t; i < E + n_chunks; i += 256) eact[i] = 0;
  }
  __syncthreads();
  for (int i = t; i < MD_BM * E; i += 256) {
    if ((rs[i] & 0x7fff) != 0) eact[i % E] = 1;   // benign race: every writer stores 1
  }
  __syncthreads();
  if (t < n_chunks) {
    const int h_lo = t * MD_HC;
    const int h_hi = (h_lo + MD_HC - 1 < hidden - 1) ? (h_lo + MD_HC - 1) : (hidden - 1);
    int any = 0;
    if (h_lo < hidden)
      for (int e = eidx[h_lo]; e <= (int)eidx[h_hi]; ++e) any |= eact[e];
    cact[t] = any;
  }
  __syncthreads();

  f32x16 acc2[2][CT];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < CT; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[a][b][r] = 0.f;

  for (int chunk = 0; chunk < n_chunks; ++chunk) {
    if (!cact[chunk]) continue;   // uniform over the workgroup
    // ------------------------------------------------ GEMM1: H^T tile of this wave
    f32x16 acc1[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc1[a][b][r] = 0.f;
    const bf16x8* ap = w1p + ((int64_t)(chunk * MD_WAVES + w) * KS1 * 2) * 64 + lane;
#pragma unroll 4
    for (int ks = 0; ks < KS1; ++ks) {
      const bf16x8 a0 = ap[(ks * 2 + 0) * 64];
      const bf16x8 a1 = ap[(ks * 2 + 1) * 64];
      const bf16x8 b0 = xs[(0 * KS1 + ks) * 64 + lane];
      const bf16x8 b1 = xs[(1 * KS1 + ks) * 64 + lane];
      acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc1[0][0], 0, 0, 0);
      acc1[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc1[0][1], 0, 0, 0);
      acc1[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc1[1][0], 0, 0, 0);
      acc1[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc1[1][1], 0, 0, 0);
    }
    // ------------------------------------------------ epilogue 1: bias, activation, mask -> h fragments in LDS
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      float bias[16];
      uint16_t ei[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int hb = chunk * MD_HC + w * 64 + rt * 32 + 8 * q + 4 * g;
        const float4 bq = *(const float4*)(b1p + hb);
        const ushort4 eq = *(const ushort4*)(eidx + hb);
        bias[q * 4 + 0] = bq.x; bias[q * 4 + 1] = bq.y; bias[q * 4 + 2] = bq.z; bias[q * 4 + 3] = bq.w;
        ei[q * 4 + 0] = eq.x; ei[q * 4 + 1] = eq.y; ei[q * 4 + 2] = eq.z; ei[q * 4 + 3] = eq.w;
      }
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const bf16_t* rrow = rs + (tt * 32 + c32) * E;
        float hv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = acc1[rt][tt][r] + bias[r];
          v = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(act_rt, v);
          v = bf16_to_f32(f32_to_bf16(v));
          hv[r] = v * bf16_to_f32(rrow[ei[r]]);
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          uint4 pk;
          pk.x = pack2_bf16(hv[half * 8 + 0], hv[half * 8 + 1]);
          pk.y = pack2_bf16(hv[half * 8 + 2], hv[half * 8 + 3]);
          pk.z = pack2_bf16(hv[half * 8 + 4], hv[half * 8 + 5]);
          pk.w = pack2_bf16(hv[half * 8 + 6], hv[half * 8 + 7]);
          const int ks2 = (w * 2 + rt) * 2 + half;
          ((uint4*)hs)[(tt * MD_KS2 + ks2) * 64 + lane] = pk;
        }
      }
    }
    __syncthreads();
    // ------------------------------------------------ GEMM2: OUT[64 tokens, D/4 columns of this wave] += H . W2
    const bf16x8* bp = w2p + ((int64_t)(chunk * MD_WAVES + w) * MD_KS2 * CT) * 64 + lane;
#pragma unroll 2
    for (int ks2 = 0; ks2 < MD_KS2; ++ks2) {
      const bf16x8 a0 = hs[(0 * MD_KS2 + ks2) * 64 + lane];
      const bf16x8 a1 = hs[(1 * MD_KS2 + ks2) * 64 + lane];
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const bf16x8 b = bp[(ks2 * CT + ct) * 64];
        acc2[0][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b, acc2[0][ct], 0, 0, 0);
        acc2[1][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b, acc2[1][ct], 0, 0, 0);
      }
    }
    __syncthreads();   // h tile is rewritten by the next chunk
  }

  // ---- final epilogue: + last_bias, + x, one rounding, store
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = w * (D / 4) + ct * 32 + c32;
    const float lb = (last_bias != nullptr) ? bf16_to_f32(last_bias[col]) : 0.f;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t n = tok0 + tt * 32 + 8 * (r / 4) + 4 * g + (r % 4);
        if (n < N) {
          float v = acc2[tt][ct][r] + lb;
          if (add_residual) v += bf16_to_f32(x[n * D + col]);
          out[n * D + col] = f32_to_bf16(v);
        }
      }
    }
  }
}

template <int D, int ACT>
static hipError_t launch_dense_cfg(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                   const void* last_bias, void* out, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  const char* base = (const char*)packed;
  constexpr int KS1 = D / 16;
  const size_t lds = (size_t)(2 * KS1 * 64 + 2 * MD_KS2 * 64) * 16 + (size_t)MD_BM * sh.n_experts * 2 +
                     (size_t)(sh.n_experts + L.n_chunks) * sizeof(int);
  if (lds > 160 * 1024) return hipErrorInvalidValue;
  auto kern = experts_mfma_dense_kernel<D, ACT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  const unsigned grid = (unsigned)cdiv64(sh.n_tokens, MD_BM);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, (const bf16_t*)x, (const bf16_t*)routing,
                     (const bf16x8*)(base + L.w1_off), (const bf16x8*)(base + L.w2_off), (const float*)(base + L.b1_off),
                     (const uint16_t*)(base + L.eidx_off), (const bf16_t*)last_bias, (bf16_t*)out, sh.n_tokens,
                     sh.n_experts, L.n_chunks, L.hidden, sh.activation, sh.add_residual);
  return hipGetLastError();
}

hipError_t launch_mfma_dense(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                             const void* last_bias, void* out, hipStream_t s) {
  switch (sh.activation) {
    case D2DMOE_ACT_RELU: return launch_dense_cfg<768, D2DMOE_ACT_RELU>(sh, x, routing, packed, last_bias, out, s);
    case D2DMOE_ACT_GELU: return launch_dense_cfg<768, D2DMOE_ACT_GELU>(sh, x, routing, packed, last_bias, out, s);
    default: return launch_dense_cfg<768, -1>(sh, x, routing, packed, last_bias, out, s);
  }
}

}  // namespace d2dmoe
