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

constexpr int MD_RING = 32;     // weight fragments kept in flight per wave (16 bytes per lane each)

struct PackedLayout {
  int hidden;      // E * Ed
  int n_chunks;    // ceil(hidden / MD_HC)
  int hidden_pad;  // n_chunks * MD_HC
  int pieces;      // weight fragments per (wave, chunk): D/16*2 for W1 followed by 16*D/128 for W2
  size_t w_off, b1_off, eidx_off, r1_off, r2_off, total;   // r1/r2: router fragments (present when routed)
  bool has_dense, has_router;
};

static size_t dense_lds_bytes(const d2dmoe_shape& sh) {
  const int hidden = sh.n_experts * sh.expert_dim;
  const int n_chunks = (hidden + MD_HC - 1) / MD_HC;
  const int KS1 = sh.d_model / 16;
  return (size_t)(2 * KS1 * 64 + 2 * MD_KS2 * 64) * 16            // x fragments, h fragments
         + (size_t)MD_BM * (sh.n_experts + 2) * 2                  // routing tile, rows padded by 2 elements
         + (size_t)n_chunks * MD_HC * 3                            // b1 (bf16) and expert index (uint8) per neuron
         + (size_t)(sh.n_experts + n_chunks + 1) * sizeof(int);    // expert-activity flags, active-chunk list
}

// The fused experts kernel is instantiated for D = 768 (ViT-B, GPT-2 small, BERT-base), ungated experts, bf16.
bool mfma_dense_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 || sh.gated) return false;
  if (sh.d_model != 768) return false;
  if (sh.n_experts > 256) return false;          // expert indices are staged as uint8
  return dense_lds_bytes(sh) <= 160 * 1024;      // x tile + h tile + routing tile + bias/expert-index tables
}

// The fused router+select kernel covers the D2DMoE router: bf16, depth 2, ReLU hidden / abs output activation,
// width and expert count both 128 or both 256, D a multiple of 16.
bool mfma_router_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 || sh.router_width <= 0) return false;
  if (sh.router_activation != D2DMOE_ACT_RELU || sh.router_output_activation != D2DMOE_ACT_ABS) return false;
  if (sh.d_model % 16 != 0) return false;
  return (sh.router_width == 128 && sh.n_experts == 128) || (sh.router_width == 256 && sh.n_experts == 256);
}

static PackedLayout packed_layout(const d2dmoe_shape& sh) {
  PackedLayout L;
  L.hidden = sh.n_experts * sh.expert_dim;
  L.n_chunks = (L.hidden + MD_HC - 1) / MD_HC;
  L.hidden_pad = L.n_chunks * MD_HC;
  L.pieces = sh.d_model / 16 * 2 + MD_KS2 * (sh.d_model / 128);
  size_t off = 0;
  L.has_dense = mfma_dense_supported(sh);
  L.w_off = off;    if (L.has_dense) off += (size_t)MD_WAVES * L.n_chunks * L.pieces * 64 * 16;
  L.b1_off = off;   if (L.has_dense) off += (size_t)L.hidden_pad * 2;   // bf16
  L.eidx_off = off; if (L.has_dense) off += (size_t)L.hidden_pad;       // uint8
  off = (off + 255) / 256 * 256;
  L.has_router = mfma_router_supported(sh);
  L.r1_off = off;   if (L.has_router) off += (size_t)sh.router_width * sh.d_model * 2;
  L.r2_off = off;   if (L.has_router) off += (size_t)sh.n_experts * sh.router_width * 2;
  L.total = (off + 255) / 256 * 256;
  return L;
}

size_t mfma_packed_bytes(const d2dmoe_shape& sh) { return packed_layout(sh).total; }

// ---------------------------------------------------------------------------------------------------
// Packing.  Each wave of the fused kernel reads ONE linear stream of 1 KB fragments (16 bytes per lane):
//   stream[wave][chunk][piece][lane][8 bf16]
//   pieces 0 .. 2*D/16-1      W1 fragments, piece = kstep*2 + rt:
//       neuron h = chunk*256 + wave*64 + rt*32 + c,  d = kstep*16 + 8g + i        value w1[h/Ed][d][h%Ed]
//   pieces 2*D/16 ..          W2 fragments, piece = 2*D/16 + ks2*(D/128) + ct:
//       neuron h = chunk*256 + (ks2/2)*32 + (ks2%2)*16 + 8*(i/4) + 4g + (i%4)
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
  const int n_w1 = D / 16 * 2;
  bf16_t v[8];
  if (piece < n_w1) {
    const int ks = piece / 2, rt = piece % 2;
    const int h = chunk * MD_HC + wave * 64 + rt * 32 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 16 + 8 * g + i;
      v[i] = (h < hidden) ? w1[((int64_t)(h / Ed) * D + d) * Ed + (h % Ed)] : (bf16_t)0;
    }
  } else {
    const int CT = D / 128;
    const int ks2 = (piece - n_w1) / CT, ct = (piece - n_w1) % CT;
    const int col = wave * (D / 4) + ct * 32 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int h = chunk * MD_HC + (ks2 / 2) * 32 + (ks2 % 2) * 16 + 8 * (i / 4) + 4 * g + (i % 4);
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
                                   bf16_t* __restrict__ d2, int D, int W, int E) {
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
      d2[pp * 8 + i] = rw2[(int64_t)(et * 32 + c) * W + wi];
    }
  }
}

hipError_t launch_mfma_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            const void* router_w1, const void* router_w2, void* packed, hipStream_t s) {
  (void)w_up;
  const PackedLayout L = packed_layout(sh);
  char* base = (char*)packed;
  if (L.has_router) {
    if (router_w1 == nullptr || router_w2 == nullptr) return hipErrorInvalidValue;
    const int64_t n = ((int64_t)sh.router_width * sh.d_model + (int64_t)sh.n_experts * sh.router_width) / 8;
    hipLaunchKernelGGL(pack_router_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)router_w1,
                       (const bf16_t*)router_w2, (bf16_t*)(base + L.r1_off), (bf16_t*)(base + L.r2_off), sh.d_model,
                       sh.router_width, sh.n_experts);
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
// Fused experts kernel, token-tile-major ("masked dense sweep").
// Workgroup = 4 waves, 64 tokens.  LDS: the x tile as B fragments (96 KB at D = 768, resident for the whole
// kernel), one chunk of h as A fragments (32 KB), the routing tile (64 x E bf16).  Per chunk of 256 neurons:
//   GEMM1  wave w: H^T[64 neurons of w, 64 tokens] over K = D        A = W1 fragments (global), B = x (LDS)
//   epilogue      + b1, activation, round to bf16, x routing[token, expert(neuron)], store as A fragments to LDS
//   GEMM2  wave w: OUT[64 tokens, D/4 columns of w] += H . W2         A = h (LDS), B = W2 fragments (global)
// OUT stays in registers across all chunks (ascending neuron = ascending expert order, float32) and is rounded
// once in the final epilogue (+ last_bias, + x).  Chunks none of whose experts is routed to by any token of the
// tile are skipped (uniform branch).
//
// Each wave runs at one wave per SIMD, so memory latency is hidden by software: the weight stream is read
// MD_RING fragments ahead into a register ring (static indices after full unrolling), across phase and chunk
// boundaries.  The two workgroup barriers per chunk wait on LDS traffic only, so the global loads in flight
// survive them; GEMM2 of chunk c and GEMM1 of the next chunk run back to back between barriers.
// ---------------------------------------------------------------------------------------------------
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two float32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ inline uint32_t pack2_bf16(float lo, float hi) {
  const f32x2 v = {lo, hi};
  const bf16x2 b = __builtin_convertvector(v, bf16x2);
  uint32_t u;
  __builtin_memcpy(&u, &b, 4);
  return u;
}

// LDS-only workgroup barrier: waits for this wave's LDS operations, not for its outstanding global loads.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int D, int ACT, bool ED8>
__global__ __launch_bounds__(256, 1) void experts_mfma_dense_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ routing, const bf16x8* __restrict__ wp,
    const bf16_t* __restrict__ b1p, const uint8_t* __restrict__ eidx, const bf16_t* __restrict__ last_bias,
    bf16_t* __restrict__ out, int64_t N, int E, int n_chunks, int hidden, int act_rt, int add_residual) {
  constexpr int KS1 = D / 16;          // K steps of GEMM1
  constexpr int CT = D / 128;          // 32-wide column tiles per wave in GEMM2
  constexpr int NW1 = KS1 * 2;         // W1 fragments per (wave, chunk)
  constexpr int NW2 = MD_KS2 * CT;     // W2 fragments per (wave, chunk)
  constexpr int PIECES = NW1 + NW2;
  constexpr int R = MD_RING;
  static_assert(NW1 % R == 0 && NW2 % R == 0, "phases must start at ring slot 0");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16x8* xs = (bf16x8*)smem_raw;                              // [2][KS1][64]
  bf16x8* hs = xs + 2 * KS1 * 64;                              // [2][MD_KS2][64]
  const int RS = E + 2;                                        // padded row stride: tokens land in different banks
  const int HP = n_chunks * MD_HC;
  bf16_t* rs = (bf16_t*)(hs + 2 * MD_KS2 * 64);                // [64][E+2] routing tile
  bf16_t* b1s = rs + MD_BM * RS;                               // [HP] first-layer bias
  int* eact = (int*)(b1s + HP);                                // [E]
  int* clist = eact + E;                                       // [n_chunks] active chunks, then their number
  int* n_act_p = clist + n_chunks;
  uint8_t* eis = (uint8_t*)(n_act_p + 1);                      // [HP] expert index of each neuron

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
      const int m = i / E, e = i - m * E;
      const int64_t n = tok0 + m;
      rs[m * RS + e] = (n < N) ? routing[n * E + e] : (bf16_t)0;
    }
    for (int i = t; i < HP / 8; i += 256) ((uint4*)b1s)[i] = ((const uint4*)b1p)[i];
    for (int i = t; i < HP / 16; i += 256) ((uint4*)eis)[i] = ((const uint4*)eidx)[i];
    for (int i = t; i < E; i += 256) eact[i] = 0;
  }
  __syncthreads();
  for (int i = t; i < MD_BM * E; i += 256) {
    const int m = i / E, e = i - m * E;
    if ((rs[m * RS + e] & 0x7fff) != 0) eact[e] = 1;   // benign race: every writer stores 1
  }
  __syncthreads();
  if (t == 0) {
    int n_act = 0;
    for (int ch = 0; ch < n_chunks; ++ch) {
      const int h_lo = ch * MD_HC;
      if (h_lo >= hidden) break;
      const int h_hi = (h_lo + MD_HC - 1 < hidden - 1) ? (h_lo + MD_HC - 1) : (hidden - 1);
      int any = 0;
      for (int e = eis[h_lo]; e <= (int)eis[h_hi]; ++e) any |= eact[e];
      if (any) clist[n_act++] = ch;
    }
    *n_act_p = n_act;
  }
  __syncthreads();
  const int n_act = *n_act_p;

  f32x16 acc2[2][CT];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < CT; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[a][b][r] = 0.f;

  if (n_act > 0) {
    const bf16x8* wbase = wp + (int64_t)w * n_chunks * PIECES * 64 + lane;   // this wave's stream
    f32x16 acc1[2][2];
    bf16x8 ring[R];

    // GEMM1 of one chunk: consumes W1 fragments 0..NW1-1 of `pre`, prefetching R fragments ahead (the stream
    // continues into the same chunk's W2 fragments).
    auto gemm1 = [&](const bf16x8* pre) {
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc1[a][b][r] = 0.f;
      bf16x8 b0 = xs[lane];
      bf16x8 b1 = xs[KS1 * 64 + lane];
#pragma unroll
      for (int ks = 0; ks < KS1; ++ks) {
        const bf16x8 a0 = ring[(2 * ks) % R];
        const bf16x8 a1 = ring[(2 * ks + 1) % R];
        ring[(2 * ks) % R] = pre[(2 * ks + R) * 64];
        ring[(2 * ks + 1) % R] = pre[(2 * ks + 1 + R) * 64];
        const int kn = (ks + 1 < KS1) ? ks + 1 : ks;      // x fragments of the next step, read one step ahead
        const bf16x8 nb0 = xs[(0 * KS1 + kn) * 64 + lane];
        const bf16x8 nb1 = xs[(1 * KS1 + kn) * 64 + lane];
        acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc1[0][0], 0, 0, 0);
        acc1[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc1[0][1], 0, 0, 0);
        acc1[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc1[1][0], 0, 0, 0);
        acc1[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc1[1][1], 0, 0, 0);
        b0 = nb0;
        b1 = nb1;
        __builtin_amdgcn_sched_barrier(0);   // keep each refill where it is written: R fragments ahead of its use
      }
    };

    const bf16x8* cur = wbase + (int64_t)clist[0] * PIECES * 64;
#pragma unroll
    for (int i = 0; i < R; ++i) ring[i] = cur[i * 64];
    gemm1(cur);

    for (int ci = 0; ci < n_act; ++ci) {
      const int chunk = clist[ci];
      const bool has_next = (ci + 1 < n_act);
      const bf16x8* nxt = has_next ? (wbase + (int64_t)clist[ci + 1] * PIECES * 64) : cur;
      // every wave has finished reading the previous h tile
      lds_barrier();
      // ---------------------------------------------- epilogue 1: bias, activation, mask -> h fragments in LDS
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        float bias[16];
        int ei[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int hb = chunk * MD_HC + w * 64 + rt * 32 + 8 * q + 4 * g;
          const uint2 bq = *(const uint2*)(b1s + hb);      // 4 bf16
          bias[q * 4 + 0] = __uint_as_float(bq.x << 16); bias[q * 4 + 1] = __uint_as_float(bq.x & 0xffff0000u);
          bias[q * 4 + 2] = __uint_as_float(bq.y << 16); bias[q * 4 + 3] = __uint_as_float(bq.y & 0xffff0000u);
          if (ED8) {
            // Ed is a multiple of 8: the aligned block of 8 neurons this q covers belongs to one expert, the same for
            // every lane, so one routing value per (q, token tile) serves four accumulator rows
            ei[q * 4] = eis[hb & ~7];
          } else {
            const uint32_t eq = *(const uint32_t*)(eis + hb);  // 4 uint8
            ei[q * 4 + 0] = eq & 0xff; ei[q * 4 + 1] = (eq >> 8) & 0xff;
            ei[q * 4 + 2] = (eq >> 16) & 0xff; ei[q * 4 + 3] = eq >> 24;
          }
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const bf16_t* rrow = rs + (tt * 32 + c32) * RS;
          float hv[16];
          float rq[4];
          if (ED8) {
#pragma unroll
            for (int q = 0; q < 4; ++q) rq[q] = bf16_to_f32(rrow[ei[q * 4]]);
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float v = acc1[rt][tt][r] + bias[r];
            v = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(act_rt, v);
            hv[r] = v * (ED8 ? rq[r / 4] : bf16_to_f32(rrow[ei[r]]));
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
      lds_barrier();   // h tile complete
      // ---------------------------------------------- GEMM2: OUT[64 tokens, D/4 columns of this wave] += H . W2
      {
        bf16x8 a0 = hs[lane];
        bf16x8 a1 = hs[MD_KS2 * 64 + lane];
#pragma unroll
        for (int ks2 = 0; ks2 < MD_KS2; ++ks2) {
          const int kn = (ks2 + 1 < MD_KS2) ? ks2 + 1 : ks2;   // h fragments of the next step, read one step ahead
          const bf16x8 na0 = hs[(0 * MD_KS2 + kn) * 64 + lane];
          const bf16x8 na1 = hs[(1 * MD_KS2 + kn) * 64 + lane];
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) {
            const int s = ks2 * CT + ct;      // position in this phase; refill position s + R
            const bf16x8 b = ring[s % R];
            ring[s % R] = (s + R < NW2) ? cur[(NW1 + s + R) * 64] : nxt[(s + R - NW2) * 64];
            acc2[0][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b, acc2[0][ct], 0, 0, 0);
            acc2[1][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b, acc2[1][ct], 0, 0, 0);
          }
          a0 = na0;
          a1 = na1;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // ---------------------------------------------- GEMM1 of the next active chunk
      if (has_next) gemm1(nxt);
      cur = nxt;
    }
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
          out[n * D + col] = (bf16_t)(pack2_bf16(v, 0.f) & 0xffffu);
        }
      }
    }
  }
}

template <int D, int ACT, bool ED8>
static hipError_t launch_dense_cfg(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                   const void* last_bias, void* out, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  const char* base = (const char*)packed;
  constexpr int KS1 = D / 16;
  const size_t lds = dense_lds_bytes(sh);
  if (lds > 160 * 1024) return hipErrorInvalidValue;
  static_assert(KS1 * 16 == D, "D must be a multiple of 16");
  auto kern = experts_mfma_dense_kernel<D, ACT, ED8>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  const unsigned grid = (unsigned)cdiv64(sh.n_tokens, MD_BM);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, (const bf16_t*)x, (const bf16_t*)routing,
                     (const bf16x8*)(base + L.w_off), (const bf16_t*)(base + L.b1_off),
                     (const uint8_t*)(base + L.eidx_off), (const bf16_t*)last_bias, (bf16_t*)out, sh.n_tokens,
                     sh.n_experts, L.n_chunks, L.hidden, sh.activation, sh.add_residual);
  return hipGetLastError();
}

template <int D, int ACT>
static hipError_t launch_dense_act(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                   const void* last_bias, void* out, hipStream_t s) {
  if (sh.expert_dim % 8 == 0) return launch_dense_cfg<D, ACT, true>(sh, x, routing, packed, last_bias, out, s);
  return launch_dense_cfg<D, ACT, false>(sh, x, routing, packed, last_bias, out, s);
}

hipError_t launch_mfma_dense(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                             const void* last_bias, void* out, hipStream_t s) {
  switch (sh.activation) {
    case D2DMOE_ACT_RELU: return launch_dense_act<768, D2DMOE_ACT_RELU>(sh, x, routing, packed, last_bias, out, s);
    case D2DMOE_ACT_GELU: return launch_dense_act<768, D2DMOE_ACT_GELU>(sh, x, routing, packed, last_bias, out, s);
    default: return launch_dense_act<768, -1>(sh, x, routing, packed, last_bias, out, s);
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
template <int WT, int ET>
__global__ __launch_bounds__(256) void router_select_mfma_kernel(
    const bf16_t* __restrict__ x, const bf16x8* __restrict__ w1f, const bf16x8* __restrict__ w2f,
    bf16_t* __restrict__ routing, bf16_t* __restrict__ norms_out, int32_t* __restrict__ counts, int64_t N, int D,
    float thr_scale) {
  constexpr int E = ET * 32;
  const int lane = threadIdx.x & 63;
  const int g = lane >> 5, c32 = lane & 31;
  const int64_t tok0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 32;
  if (tok0 >= N) return;   // whole wave; the kernel has no barriers
  const int64_t token = tok0 + c32;
  const bool valid = token < N;
  const bf16x8* xrow = (const bf16x8*)(x + (valid ? token : (N - 1)) * D);
  const int KS1 = D / 16;

  f32x16 acc1[WT];
#pragma unroll
  for (int a = 0; a < WT; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[a][r] = 0.f;
  for (int ks = 0; ks < KS1; ++ks) {
    const bf16x8 b = xrow[2 * ks + g];
#pragma unroll
    for (int rt = 0; rt < WT; ++rt) {
      const bf16x8 a = w1f[(int64_t)(ks * WT + rt) * 64 + lane];
      acc1[rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc1[rt], 0, 0, 0);
    }
  }
  // hidden activations as B fragments of the second product
  bf16x8 hb[2 * WT];
#pragma unroll
  for (int rt = 0; rt < WT; ++rt)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint4 pk;
      pk.x = pack2_bf16(fmaxf(acc1[rt][half * 8 + 0], 0.f), fmaxf(acc1[rt][half * 8 + 1], 0.f));
      pk.y = pack2_bf16(fmaxf(acc1[rt][half * 8 + 2], 0.f), fmaxf(acc1[rt][half * 8 + 3], 0.f));
      pk.z = pack2_bf16(fmaxf(acc1[rt][half * 8 + 4], 0.f), fmaxf(acc1[rt][half * 8 + 5], 0.f));
      pk.w = pack2_bf16(fmaxf(acc1[rt][half * 8 + 6], 0.f), fmaxf(acc1[rt][half * 8 + 7], 0.f));
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
      acc2[et] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, hb[ks2], acc2[et], 0, 0, 0);
    }
  }
  // norms (bf16 values held as float), per-token maximum
  float m = -INFINITY;
#pragma unroll
  for (int et = 0; et < ET; ++et)
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const uint32_t pk = pack2_bf16(fabsf(acc2[et][r]), fabsf(acc2[et][r + 1]));
      acc2[et][r] = __uint_as_float(pk << 16);
      acc2[et][r + 1] = __uint_as_float(pk & 0xffff0000u);
      m = nanmax(m, nanmax(acc2[et][r], acc2[et][r + 1]));
    }
  m = nanmax(m, __shfl_xor(m, 32, kWave));
  const float thr = __uint_as_float(pack2_bf16(m * thr_scale, 0.f) << 16);
#pragma unroll
  for (int et = 0; et < ET; ++et) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e0 = et * 32 + 8 * q + 4 * g;
      bool on[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) on[s] = acc2[et][q * 4 + s] >= thr;
      if (valid) {
        uint2 rv;
        rv.x = (on[0] ? 0x3F80u : 0u) | (on[1] ? 0x3F800000u : 0u);   // bf16 1.0 = 0x3F80
        rv.y = (on[2] ? 0x3F80u : 0u) | (on[3] ? 0x3F800000u : 0u);
        *(uint2*)(routing + token * E + e0) = rv;
        if (norms_out != nullptr) {
          uint2 nv;
          nv.x = (__float_as_uint(acc2[et][q * 4 + 0]) >> 16) | (__float_as_uint(acc2[et][q * 4 + 1]) & 0xffff0000u);
          nv.y = (__float_as_uint(acc2[et][q * 4 + 2]) >> 16) | (__float_as_uint(acc2[et][q * 4 + 3]) & 0xffff0000u);
          *(uint2*)(norms_out + token * E + e0) = nv;
        }
      }
      if (counts != nullptr) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const unsigned long long bal = __ballot(on[s] && valid);
          if (lane == 0) {
            const int lo = __popcll(bal & 0xffffffffull), hi = __popcll(bal >> 32);
            if (lo) atomicAdd(counts + et * 32 + 8 * q + s, lo);
            if (hi) atomicAdd(counts + et * 32 + 8 * q + 4 + s, hi);
          }
        }
      }
    }
  }
}

hipError_t launch_mfma_router_select(const d2dmoe_shape& sh, const void* x, const void* packed, void* routing,
                                     void* norms_out, int32_t* counts, float thr_scale, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  if (!L.has_router) return hipErrorInvalidValue;
  const char* base = (const char*)packed;
  if (counts != nullptr) {
    hipError_t e = launch_fill_i32(counts, sh.n_experts, 0, s);
    if (e != hipSuccess) return e;
  }
  const unsigned grid = (unsigned)cdiv64(sh.n_tokens, 128);
  if (sh.router_width == 128)
    hipLaunchKernelGGL((router_select_mfma_kernel<4, 4>), dim3(grid), dim3(256), 0, s, (const bf16_t*)x,
                       (const bf16x8*)(base + L.r1_off), (const bf16x8*)(base + L.r2_off), (bf16_t*)routing,
                       (bf16_t*)norms_out, counts, sh.n_tokens, sh.d_model, thr_scale);
  else
    hipLaunchKernelGGL((router_select_mfma_kernel<8, 8>), dim3(grid), dim3(256), 0, s, (const bf16_t*)x,
                       (const bf16x8*)(base + L.r1_off), (const bf16x8*)(base + L.r2_off), (bf16_t*)routing,
                       (bf16_t*)norms_out, counts, sh.n_tokens, sh.d_model, thr_scale);
  return hipGetLastError();
}

}  // namespace d2dmoe
