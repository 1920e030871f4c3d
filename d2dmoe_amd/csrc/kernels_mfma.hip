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
  size_t w_off, b1_off, eidx_off, total;
};

static PackedLayout packed_layout(const d2dmoe_shape& sh) {
  PackedLayout L;
  L.hidden = sh.n_experts * sh.expert_dim;
  L.n_chunks = (L.hidden + MD_HC - 1) / MD_HC;
  L.hidden_pad = L.n_chunks * MD_HC;
  L.pieces = sh.d_model / 16 * 2 + MD_KS2 * (sh.d_model / 128);
  size_t off = 0;
  L.w_off = off;    off += (size_t)MD_WAVES * L.n_chunks * L.pieces * 64 * 16;
  L.b1_off = off;   off += (size_t)L.hidden_pad * 2;   // bf16
  L.eidx_off = off; off += (size_t)L.hidden_pad;       // uint8
  L.total = (off + 255) / 256 * 256;
  return L;
}

static size_t dense_lds_bytes(const d2dmoe_shape& sh) {
  const PackedLayout L = packed_layout(sh);
  const int KS1 = sh.d_model / 16;
  return (size_t)(2 * KS1 * 64 + 2 * MD_KS2 * 64) * 16            // x fragments, h fragments
         + (size_t)MD_BM * (sh.n_experts + 2) * 2                  // routing tile, rows padded by 2 elements
         + (size_t)L.hidden_pad * 3                                // b1 (bf16) and expert index (uint8) per neuron
         + (size_t)(sh.n_experts + L.n_chunks + 1) * sizeof(int);  // expert-activity flags, active-chunk list
}

bool mfma_dense_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 || sh.gated) return false;
  if (sh.d_model != 768) return false;
  if (sh.n_experts > 256) return false;          // expert indices are staged as uint8
  return dense_lds_bytes(sh) <= 160 * 1024;      // x tile + h tile + routing tile + bias/expert-index tables
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

hipError_t launch_mfma_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            const void* router_w1, const void* router_w2, void* packed, hipStream_t s) {
  (void)w_up; (void)router_w1; (void)router_w2;
  const PackedLayout L = packed_layout(sh);
  char* base = (char*)packed;
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

template <int D, int ACT>
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
          const uint32_t eq = *(const uint32_t*)(eis + hb);  // 4 uint8
          bias[q * 4 + 0] = __uint_as_float(bq.x << 16); bias[q * 4 + 1] = __uint_as_float(bq.x & 0xffff0000u);
          bias[q * 4 + 2] = __uint_as_float(bq.y << 16); bias[q * 4 + 3] = __uint_as_float(bq.y & 0xffff0000u);
          ei[q * 4 + 0] = eq & 0xff; ei[q * 4 + 1] = (eq >> 8) & 0xff;
          ei[q * 4 + 2] = (eq >> 16) & 0xff; ei[q * 4 + 3] = eq >> 24;
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const bf16_t* rrow = rs + (tt * 32 + c32) * RS;
          float hv[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float v = acc1[rt][tt][r] + bias[r];
            v = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(act_rt, v);
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

template <int D, int ACT>
static hipError_t launch_dense_cfg(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                   const void* last_bias, void* out, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  const char* base = (const char*)packed;
  constexpr int KS1 = D / 16;
  const size_t lds = dense_lds_bytes(sh);
  if (lds > 160 * 1024) return hipErrorInvalidValue;
  static_assert(KS1 * 16 == D, "D must be a multiple of 16");
  auto kern = experts_mfma_dense_kernel<D, ACT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  const unsigned grid = (unsigned)cdiv64(sh.n_tokens, MD_BM);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, (const bf16_t*)x, (const bf16_t*)routing,
                     (const bf16x8*)(base + L.w_off), (const bf16_t*)(base + L.b1_off),
                     (const uint8_t*)(base + L.eidx_off), (const bf16_t*)last_bias, (bf16_t*)out, sh.n_tokens,
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
