// Small-batch ("decode") bf16 MFMA path: at most 16 tokens, so the layer is bound by streaming the weights of the
// routed experts once.  One workgroup per expert pulls that expert's packed gate/up weights through
// v_mfma_f32_16x16x32_bf16 with all tokens resident in LDS and leaves the hidden activations (256 KB for 256 experts
// of 32 neurons) in memory; a second kernel owns 16 output columns per workgroup and sums the down projections of the
// routed experts in ascending order.  Also here: a skinny Linear kernel (router layers for <= 16 tokens) that needs no packing.
//
// Fragment layouts of the 16x16x32 bf16 MFMA on a 64-lane wave (gq = lane / 16, c = lane % 16):
//   A (16 x 32): lane holds row c,    k = 8 gq .. 8 gq + 7
//   B (32 x 16): lane holds column c, k = 8 gq .. 8 gq + 7
//   C (16 x 16): lane holds column c, rows 4 gq + r for r = 0..3
// As in the large-batch kernels the first product is computed transposed (H^T = W^T . X^T), which leaves every lane
// holding ONE token and, over two 16-neuron tiles, the 8 values one B fragment of the second product needs; the
// implied k order (slot (gq, i) <-> neuron 16*(i/4) + 4 gq + (i%4) of a 32-block) is baked into the packed W2^T
// fragments.
#include "mfma_common.hpp"

namespace d2dmoe {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int DC_MAX_TOKENS = 16;

struct DecodeLayout {
  int edp;      // neurons per expert padded to a multiple of 32
  int nt16;     // 16-neuron tiles per expert
  size_t gu_off, d_off, b_off, total;   // gate(/up) fragment stream, down^T fragments, bias (bf16, padded)
};

static DecodeLayout decode_layout(const d2dmoe_shape& sh) {
  DecodeLayout L;
  L.edp = (sh.expert_dim + 31) / 32 * 32;
  L.nt16 = L.edp / 16;
  const size_t mat = (size_t)sh.n_experts * L.edp * sh.d_model * 2;
  size_t off = 0;
  L.gu_off = off; off += mat * (sh.gated ? 2 : 1);
  L.d_off = off; off += mat;
  L.b_off = off; off += (size_t)sh.n_experts * L.edp * 2;
  L.total = (off + 255) / 256 * 256;
  return L;
}

bool mfma_decode_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 && sh.dtype != D2DMOE_F16) return false;
  if (sh.d_model % 256 != 0 || sh.d_model > 4096) return false;   // an even number of whole 32-steps per wave
  const int edp = (sh.expert_dim + 31) / 32 * 32;
  return edp == 32 || edp == 64 || edp == 128;
}

size_t mfma_decode_packed_bytes(const d2dmoe_shape& sh) { return mfma_decode_supported(sh) ? decode_layout(sh).total : 0; }

size_t mfma_decode_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_decode_supported(sh)) return 0;
  // hidden activations as bf16 fragments, then one "some token routes here" flag per expert
  return (size_t)sh.n_experts * decode_layout(sh).edp * DC_MAX_TOKENS * 2 + (size_t)sh.n_experts * 4;
}

// ---------------------------------------------------------------------------------------------------
// Packing.  KS = D/32 K steps, EdP padded neurons, NB = EdP/32 neuron blocks, NM = 2 if gated else 1.  Every workgroup of
// the two kernels below reads ONE contiguous stream.
//   gate(/up) stream [E][block NB][kstep KS][matrix NM][tile 2][lane 64][8]:
//                    neuron j = block*32 + tile*16 + c, d = kstep*32 + 8 gq + i                          w[e][d][j]
//   down^T stream    [column block D/8][E][kstep2 NB][gq 4][c8 8][8]:  column = cb*8 + c8,
//                    neuron j = ks2*32 + 16*(i/4) + 4 gq + (i%4)                                         w2[e][j][column]
//   bias             [E][EdP] bf16
// ---------------------------------------------------------------------------------------------------
__global__ void pack_decode_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ b1, const bf16_t* __restrict__ w2,
                                   const bf16_t* __restrict__ w_up, bf16_t* __restrict__ dgu, bf16_t* __restrict__ dd,
                                   bf16_t* __restrict__ db, int D, int E, int Ed, int edp) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int nm = (w_up != nullptr) ? 2 : 1;
  const int KS = D / 32, NB = edp / 32;
  const int64_t n_gu = (int64_t)E * NB * KS * nm * 2 * 64;   // 16-byte pieces
  const int64_t n_d = (int64_t)(D / 8) * E * NB * 32;
  if (p < n_gu) {
    int64_t q = p;
    const int lane = (int)(q % 64); q /= 64;
    const int tile = (int)(q % 2); q /= 2;
    const int m = (int)(q % nm); q /= nm;
    const int ks = (int)(q % KS); q /= KS;
    const int blk = (int)(q % NB);
    const int e = (int)(q / NB);
    const int gq = lane / 16, c = lane % 16;
    const bf16_t* src = m ? w_up : w1;
    const int j = blk * 32 + tile * 16 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 32 + 8 * gq + i;
      dgu[p * 8 + i] = (j < Ed) ? src[((int64_t)e * D + d) * Ed + j] : (bf16_t)0;
    }
  } else if (p < n_gu + n_d) {
    const int64_t pp = p - n_gu;
    int64_t q = pp;
    const int c8 = (int)(q % 8); q /= 8;
    const int gq = (int)(q % 4); q /= 4;
    const int ks2 = (int)(q % NB); q /= NB;
    const int e = (int)(q % E);
    const int cb = (int)(q / E);
    const int col = cb * 8 + c8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = ks2 * 32 + 16 * (i / 4) + 4 * gq + (i % 4);
      dd[pp * 8 + i] = (j < Ed) ? w2[((int64_t)e * Ed + j) * D + col] : (bf16_t)0;
    }
  } else if (p < n_gu + n_d + (int64_t)E * edp) {
    const int64_t pp = p - n_gu - n_d;
    const int e = (int)(pp / edp), j = (int)(pp % edp);
    db[pp] = (j < Ed && b1 != nullptr) ? b1[(int64_t)e * Ed + j] : (bf16_t)0;
  }
}

hipError_t launch_decode_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                              void* packed_section, hipStream_t s) {
  const DecodeLayout L = decode_layout(sh);
  char* base = (char*)packed_section;
  const int nm = sh.gated ? 2 : 1;
  const int64_t n = (int64_t)(nm + 1) * sh.n_experts * L.edp * sh.d_model / 8 + (int64_t)sh.n_experts * L.edp;
  hipLaunchKernelGGL(pack_decode_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)w1, (const bf16_t*)b1,
                     (const bf16_t*)w2, sh.gated ? (const bf16_t*)w_up : (const bf16_t*)nullptr, (bf16_t*)(base + L.gu_off),
                     (bf16_t*)(base + L.d_off), (bf16_t*)(base + L.b_off), sh.d_model, sh.n_experts, sh.expert_dim, L.edp);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Two kernels, no per-expert output rows in memory:
//
// decode_hidden_kernel: workgroup = (expert, block of 32 neurons), 4 waves.
//   leave at once if no token routes to the expert
//   GEMM1   wave w: its quarter of K for the block's two neuron tiles, gate and (if gated) up.  Weight fragments and
//           the x fragments (straight from the row-major x, which stays in L2) go through two register buffers so the
//           stream never drains; the four partial tiles are summed through LDS in wave order
//   hidden  gated: act(g) * u, else act(g + b1); times the routing weight; rounded to bf16 and stored as one B
//           fragment of the second product: hfrag[e][block][lane]
//
// decode_out_kernel: workgroup = 8 output columns, 8 waves.
//   the routed experts are listed in ascending order and cut into 8 consecutive runs, one per wave; a wave chains
//   OUT^T += W2[e]^T . H[e]^T over its run in one float32 accumulator (rows 8..15 of the 16-row MFMA tile repeat
//   rows 0..7 and are dropped); the 8 partial tiles are added in wave order, then last_bias and the residual, one
//   rounding.  The summation order depends on the routing only.
// ---------------------------------------------------------------------------------------------------
struct DecodeArgs {
  const bf16_t* x; const bf16_t* routing; const bf16x8* wgu; const bf16x8* wd; const bf16_t* bias;
  bf16x8* hfrag; int* active; const bf16_t* last_bias; bf16_t* out; int N; int D; int E; int nt16; int act; int add_residual;
  // Whole layer in three launches (fused != 0): the hidden kernel computes every expert (it does not wait for the routing)
  // and its extra workgroups compute the first router layer; the output kernel derives the routing from the norms itself.
  int fused;
  const bf16_t* rw1; bf16_t* rhidden; int rwidth; int ract;     // first router layer: [rwidth, D] -> rhidden [N, rwidth]
  const bf16_t* norms; bf16_t* routing_out; int32_t* counts; float thr_scale;
};

// First router layer inside the hidden kernel's launch: 4 features per workgroup of 4 waves.  K is cut into the same parts
// as by linear_skinny_kernel (16 where K is long, else 4), each part accumulated on its own in K order and the parts
// summed in order, so the result has the bits that kernel produces.
template <bool F16>
__device__ __forceinline__ void decode_router_l1_block(const DecodeArgs& A, int blk, float (*part)[4][64]) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int gq = lane >> 4, c16 = lane & 15;
  const int K = A.D, Nout = A.rwidth, N = A.N;
  const int P = (K % 512 == 0 && K >= 1024) ? 16 : 4;   // parts of K
  const int KQ = K / P;                                   // a multiple of 32
  const int f0 = blk * 4;
  const int fr = f0 + (c16 & 3);
  const int frow = (fr < Nout) ? fr : (Nout - 1);
  const int trow = (c16 < N) ? c16 : (N - 1);
  for (int p = w * (P / 4); p < (w + 1) * (P / 4); ++p) {
    const bf16x8* bp = (const bf16x8*)(A.rw1 + (int64_t)frow * K + p * KQ) + gq;
    const bf16x8* ap = (const bf16x8*)(A.x + (int64_t)trow * K + p * KQ) + gq;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int ks0 = 0; ks0 < KQ / 32; ks0 += 4) {
      bf16x8 bv[4], av[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int ks = (ks0 + u < KQ / 32) ? (ks0 + u) : ks0;
        bv[u] = bp[ks * 4];
        av[u] = ap[ks * 4];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (ks0 + u < KQ / 32) acc = mfma_16x16x32<F16>(bv[u], av[u], acc);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) part[p][r][lane] = acc[r];
  }
  __syncthreads();
  if (w == 0 && gq == 0 && c16 < N) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = part[0][r][lane];
      for (int pp = 1; pp < P; ++pp) v += part[pp][r][lane];
      const int f = f0 + r;
      if (f < Nout) {
        const float vr = round16<F16>(v);
        A.rhidden[(int64_t)c16 * Nout + f] = enc16<F16>(apply_act(A.ract, vr));
      }
    }
  }
}

template <bool GATED, int U1, bool F16 = false>
__global__ __launch_bounds__(256) void decode_hidden_kernel(const DecodeArgs A) {
  __shared__ float part_raw[16 * 4 * 64];          // [4][NM * 8][64] here, [16][4][64] for the router workgroups
  float (*part)[(GATED ? 2 : 1) * 8][64] = (float (*)[(GATED ? 2 : 1) * 8][64])part_raw;
  const int D = A.D, N = A.N, E = A.E, NT16 = A.nt16;
  // fused: the first workgroups of the grid are the router's (they start first, so the second router layer's input is
  // ready long before the grid has drained)
  const int n_router = A.fused ? (A.rwidth + 3) / 4 : 0;
  if ((int)blockIdx.x < n_router) {
    decode_router_l1_block<F16>(A, (int)blockIdx.x, (float (*)[4][64])part_raw);
    return;
  }
  const int hb = (int)blockIdx.x - n_router;
  const int KS = D / 32;          // K steps of GEMM1
  const int KQ = KS / 4;          // per wave
  constexpr int NM = GATED ? 2 : 1;
  constexpr int FPS = NM * 2;     // fragments per K step
  const int KS2 = NT16 / 2;
  const int e = hb / KS2, k2 = hb % KS2;
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int gq = lane >> 4, c16 = lane & 15;
  const int tc = (c16 < N) ? c16 : (N - 1);
  const bf16_t rbits = A.fused ? (bf16_t)(F16 ? 0x3c00 : 0x3f80) : A.routing[(int64_t)tc * E + e];   // fused: the routing is applied later
  const bool any = __ballot((rbits & 0x7fff) != 0) != 0ull;
  if (!A.fused && k2 == 0 && t == 0) A.active[e] = any ? 1 : 0;
  if (!any) return;   // nobody routes to this expert: its fragments are never read

  f32x4 acc1[NM][2];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int a = 0; a < 2; ++a) acc1[m][a] = f32x4{0.f, 0.f, 0.f, 0.f};
  // this workgroup's stream is contiguous: KS steps of FPS fragments; wave w takes steps [w*KQ, (w+1)*KQ)
  const bf16x8* wf = A.wgu + ((int64_t)hb * KS + (int64_t)w * KQ) * FPS * 64 + lane;
  const bf16x8* xf = (const bf16x8*)(A.x + (int64_t)tc * D + (int64_t)w * KQ * 32) + gq;   // + 4 per K step
  // Two register buffers of U1 K steps each: while one is multiplied the other is being filled.  KQ is a multiple of
  // 2*U1 (the launcher picks U1 that way).
  bf16x8 wA[U1][FPS], xA[U1], wB[U1][FPS], xB[U1];
  auto fill = [&](bf16x8 (&wr)[U1][FPS], bf16x8 (&xb)[U1], int ks0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U1; ++u) {
      xb[u] = xf[(ks0 + u) * 4];
#pragma unroll
      for (int f = 0; f < FPS; ++f) wr[u][f] = wf[((ks0 + u) * FPS + f) * 64];
    }
  };
  auto multiply = [&](bf16x8 (&wr)[U1][FPS], bf16x8 (&xb)[U1]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U1; ++u)
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int a = 0; a < 2; ++a)
          acc1[m][a] = mfma_16x16x32<F16>(wr[u][m * 2 + a], xb[u], acc1[m][a]);
  };
  fill(wA, xA, 0);
  for (int ks0 = 0; ks0 < KQ; ks0 += 2 * U1) {
    fill(wB, xB, ks0 + U1);
    multiply(wA, xA);
    fill(wA, xA, (ks0 + 2 * U1 < KQ) ? (ks0 + 2 * U1) : ks0);   // the last trip re-reads its own steps: in bounds, unused
    multiply(wB, xB);
  }
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int r = 0; r < 4; ++r) part[w][m * 8 + a * 4 + r][lane] = acc1[m][a][r];
  __syncthreads();
  if (w != 0) return;
  // ---- hidden activations -> the block's B fragment of GEMM2.  Rows of x beyond N were copies of row N-1; their
  // columns are zeroed here and never stored by the output kernel.
  const float rw = (c16 < N) ? dec16<F16>(rbits) : 0.f;
  const bf16_t* bias_e = A.bias + (int64_t)e * NT16 * 16 + k2 * 32;
  float hv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int a = i >> 2, r = i & 3;
    float gsum = 0.f, usum = 0.f;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) {
      gsum += part[ww][a * 4 + r][lane];
      if (GATED) usum += part[ww][(NM - 1) * 8 + a * 4 + r][lane];
    }
    float v;
    if (GATED) {
      v = apply_act(A.act, gsum) * usum;
    } else {
      v = apply_act(A.act, gsum + dec16<F16>(bias_e[a * 16 + 4 * gq + r]));
    }
    hv[i] = (c16 < N) ? v * rw : 0.f;
  }
  uint4 pk;
  pk.x = enc16x2<F16>(hv[0], hv[1]); pk.y = enc16x2<F16>(hv[2], hv[3]);
  pk.z = enc16x2<F16>(hv[4], hv[5]); pk.w = enc16x2<F16>(hv[6], hv[7]);
  ((uint4*)A.hfrag)[((int64_t)e * KS2 + k2) * 64 + lane] = pk;
}

constexpr int DO_WAVES = 8;

// Workgroup = 8 output columns, 8 waves; wave w owns experts [w*EW, (w+1)*EW) with EW = ceil(E/8) rounded up to 64 at
// most per pass, and walks the routed ones among them in ascending order.
template <int KS2, bool F16 = false>
__global__ __launch_bounds__(DO_WAVES * 64) void decode_out_kernel(const DecodeArgs A) {
  constexpr int UB = 8 / KS2;                  // experts per load batch (8 hidden fragments, half as many weight loads;
                                               // twice as many in flight was slower: 18.7 against 16.7 us at 16 tokens)
  __shared__ float part[DO_WAVES][4][64];
  __shared__ float s_thr[16];                  // fused: the tokens' thresholds
  __shared__ unsigned short s_bits[DO_WAVES * 64];   // fused: per expert, bit t = token t routes to it
  const int D = A.D, N = A.N, E = A.E;
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int gq = lane >> 4, c16 = lane & 15;
  const int cb = blockIdx.x;                   // 8-column block
  const int EW = (E + DO_WAVES - 1) / DO_WAVES;
  const int e_lo = w * EW, e_hi = (e_lo + EW < E) ? (e_lo + EW) : E;
  if (A.fused) {
    // Dynamic-k selection from the norms (moefication.py:80-85), by every workgroup for itself (8 KB out of L2): wave 0
    // takes the maximum of every token's row, then a lane per expert compares its column with the thresholds.  Same
    // arithmetic as select_kernel: m NaN-propagating, thr = round(m * thr_scale), on = norm >= thr.
    // (E <= 512 here: one expert per thread; its column is requested before the maxima are worked out)
    const int ecol = (t < E) ? t : (E - 1);
    bf16_t colv[DC_MAX_TOKENS];
#pragma unroll
    for (int tk = 0; tk < DC_MAX_TOKENS; ++tk) colv[tk] = A.norms[(int64_t)(tk < N ? tk : N - 1) * E + ecol];
    if (w == 0) {
      const int tc = (c16 < N) ? c16 : (N - 1);
      float m = -INFINITY;
      for (int e8 = gq * 8; e8 < E; e8 += 32) {          // E is a multiple of 32 here
        const u32x4 v = *(const u32x4*)(A.norms + (int64_t)tc * E + e8);
        const uint32_t vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) m = nanmax(m, (i & 1) ? dec16_hi<F16>(vw[i >> 1]) : dec16<F16>(vw[i >> 1] & 0xffffu));
      }
      m = nanmax(m, __shfl_xor(m, 16, 64));
      m = nanmax(m, __shfl_xor(m, 32, 64));
      // (the product is rounded to float32 before it is rounded to the storage type: kept apart by the empty asm, or the
      // compiler folds multiply and float16 conversion into one instruction with a single rounding)
      float thr_prod = m * A.thr_scale;
      asm volatile("" : "+v"(thr_prod));
      if (gq == 0) s_thr[c16] = round16<F16>(thr_prod);
    }
    __syncthreads();
    if (t < E) {
      unsigned bits = 0u;
#pragma unroll
      for (int tk = 0; tk < DC_MAX_TOKENS; ++tk) bits |= ((tk < N && dec16<F16>(colv[tk]) >= s_thr[tk]) ? 1u : 0u) << tk;
      s_bits[t] = (unsigned short)bits;
      if (cb == 0) {                                      // one workgroup also leaves the routing tensor and the counts
        for (int tk = 0; tk < N; ++tk) A.routing_out[(int64_t)tk * E + t] = ((bits >> tk) & 1u) ? (bf16_t)(F16 ? 0x3c00 : 0x3f80) : (bf16_t)0;
        if (A.counts != nullptr) A.counts[t] = __popc(bits);
      }
    }
    __syncthreads();
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  // A fragment rows 0..7 only (lanes c16 >= 8 repeat them); result rows 8..15 are dropped
  const bf16x8* wdf = A.wd + (int64_t)cb * E * KS2 * 32 + gq * 8 + (c16 & 7);
  const bf16x8* hf = A.hfrag + lane;
  constexpr int KP = (KS2 + 1) / 2;            // weight loads per expert: two K steps each
  const int khalf = (KS2 > 1) ? (c16 >> 3) : 0;
  bf16x8 aA[UB][KP], bA[UB][KS2], aB[UB][KP], bB[UB][KS2];
  int esA[UB], esB[UB];
  for (int e0 = e_lo; e0 < e_hi; e0 += 64) {   // 64 experts per pass: one flag per lane
    const bool on = (e0 + lane < e_hi) && (A.fused ? (s_bits[e0 + lane] != 0) : (A.active[e0 + lane] != 0));
    unsigned long long mask = __ballot(on);
    int cntA = 0, cntB = 0;
    // take the next up to UB routed experts off the mask and request their fragments; unused slots repeat the last one
    auto fill = [&](bf16x8 (&a)[UB][KP], bf16x8 (&b)[UB][KS2], int (&es)[UB], int& cnt) __attribute__((always_inline)) {
      cnt = 0;
      int e = e0;
#pragma unroll
      for (int j = 0; j < UB; ++j) {
        if (mask != 0ull) {
          e = e0 + (int)__builtin_ctzll(mask);
          mask &= mask - 1ull;
          ++cnt;
        }
#pragma unroll
        for (int k2 = 0; k2 < KS2; ++k2) b[j][k2] = hf[((int64_t)e * KS2 + k2) * 64];
        es[j] = e;
      }
      // Rows 8..15 of the A tile are not needed (the result rows they produce are dropped), so their lanes fetch the
      // fragment of the NEXT K step instead of repeating rows 0..7: one load brings two K steps, and the second one's
      // MFMA takes the register rotated by 8 lanes inside every row of 16 (a DPP move).  No load sits under a
      // lane-dependent branch.  (KS2 == 1: nothing to pair, the upper lanes repeat the lower ones.)
#pragma unroll
      for (int j = 0; j < UB; ++j)
#pragma unroll
        for (int kp = 0; kp < KP; ++kp) a[j][kp] = wdf[((int64_t)es[j] * KS2 + 2 * kp + khalf) * 32];
    };
    auto multiply = [&](bf16x8 (&a)[UB][KP], bf16x8 (&b)[UB][KS2], int (&es)[UB], int cnt) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < UB; ++j) {
        if (j < cnt) {
          // fused: the hidden fragment holds every token; the columns of tokens that do not route here are cleared
          const bool keep = A.fused ? (((s_bits[es[j]] >> c16) & 1u) != 0u) : true;
#pragma unroll
          for (int k2 = 0; k2 < KS2; ++k2) {
            u32x4 bm = __builtin_bit_cast(u32x4, b[j][k2]);
            bm.x = keep ? bm.x : 0u; bm.y = keep ? bm.y : 0u; bm.z = keep ? bm.z : 0u; bm.w = keep ? bm.w : 0u;
            bf16x8 av = a[j][k2 / 2];
            if (KS2 > 1 && (k2 & 1)) {       // the odd K step sits in the upper 8 lanes of every row: rotate it down
              u32x4 aw = __builtin_bit_cast(u32x4, av);
              aw.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)aw.x, 0x128, 0xf, 0xf, false);
              aw.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)aw.y, 0x128, 0xf, 0xf, false);
              aw.z = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)aw.z, 0x128, 0xf, 0xf, false);
              aw.w = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)aw.w, 0x128, 0xf, 0xf, false);
              av = __builtin_bit_cast(bf16x8, aw);
            }
            acc = mfma_16x16x32<F16>(av, __builtin_bit_cast(bf16x8, bm), acc);
          }
        }
      }
    };
    if (mask != 0ull) {
      fill(aA, bA, esA, cntA);
      while (cntA > 0) {
        cntB = 0;
        if (mask != 0ull) fill(aB, bB, esB, cntB);
        multiply(aA, bA, esA, cntA);
        cntA = 0;
        if (mask != 0ull) fill(aA, bA, esA, cntA);
        multiply(aB, bB, esB, cntB);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) part[w][r][lane] = acc[r];
  __syncthreads();
  if (w == 0 && c16 < N && gq < 2) {
    // C layout (transposed product): lane holds token c16, rows 4 gq + r = columns cb*8 + 4 gq + r
    float o[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sacc = part[0][r][lane];
#pragma unroll
      for (int ww = 1; ww < DO_WAVES; ++ww) sacc += part[ww][r][lane];
      o[r] = sacc;
    }
    const int col = cb * 8 + 4 * gq;
    if (A.last_bias != nullptr) {
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] += dec16<F16>(A.last_bias[col + r]);
    }
    if (A.add_residual) {
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] += dec16<F16>(A.x[(int64_t)c16 * D + col + r]);
    }
    uint2 ov;
    ov.x = enc16x2<F16>(o[0], o[1]);
    ov.y = enc16x2<F16>(o[2], o[3]);
    *(uint2*)(A.out + (int64_t)c16 * D + col) = ov;
  }
}

template <bool GATED, bool F16>
static hipError_t launch_hidden(const DecodeArgs& A, hipStream_t s) {
  // K steps per wave (D/128) must be a multiple of 2*U1; D is a multiple of 256, so U1 = 1 always fits.
  const int KQ = A.D / 128;
  const dim3 grid((unsigned)(A.E * (A.nt16 / 2) + (A.fused ? (A.rwidth + 3) / 4 : 0)));
  if (KQ % 8 == 0) hipLaunchKernelGGL((decode_hidden_kernel<GATED, 4, F16>), grid, dim3(256), 0, s, A);
  else if (KQ % 4 == 0) hipLaunchKernelGGL((decode_hidden_kernel<GATED, 2, F16>), grid, dim3(256), 0, s, A);
  else hipLaunchKernelGGL((decode_hidden_kernel<GATED, 1, F16>), grid, dim3(256), 0, s, A);
  return hipGetLastError();
}

// both kernels of the experts for one storage type
template <bool F16>
static hipError_t launch_hidden_t(const DecodeArgs& A, bool gated, hipStream_t s) {
  return gated ? launch_hidden<true, F16>(A, s) : launch_hidden<false, F16>(A, s);
}
template <bool F16>
static void launch_out_t(const DecodeArgs& A, int nt16, unsigned grid, hipStream_t s) {
  if (nt16 == 2) hipLaunchKernelGGL((decode_out_kernel<1, F16>), dim3(grid), dim3(DO_WAVES * 64), 0, s, A);
  else if (nt16 == 4) hipLaunchKernelGGL((decode_out_kernel<2, F16>), dim3(grid), dim3(DO_WAVES * 64), 0, s, A);
  else hipLaunchKernelGGL((decode_out_kernel<4, F16>), dim3(grid), dim3(DO_WAVES * 64), 0, s, A);
}

hipError_t launch_mfma_decode(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                              const void* last_bias, void* out, void* workspace, hipStream_t s) {
  const DecodeLayout L = decode_layout(sh);
  const char* pk = (const char*)packed_section;
  DecodeArgs A;
  A.x = (const bf16_t*)x; A.routing = (const bf16_t*)routing; A.wgu = (const bf16x8*)(pk + L.gu_off);
  A.wd = (const bf16x8*)(pk + L.d_off); A.bias = (const bf16_t*)(pk + L.b_off);
  A.hfrag = (bf16x8*)workspace;
  A.active = (int*)((char*)workspace + (size_t)sh.n_experts * L.edp * DC_MAX_TOKENS * 2);
  A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out;
  A.N = (int)sh.n_tokens; A.D = sh.d_model; A.E = sh.n_experts; A.nt16 = L.nt16; A.act = sh.activation;
  A.add_residual = sh.add_residual;
  A.fused = 0; A.rw1 = nullptr; A.rhidden = nullptr; A.rwidth = 0; A.ract = 0; A.norms = nullptr; A.routing_out = nullptr;
  A.counts = nullptr; A.thr_scale = 0.f;
  const bool f16 = sh.dtype == D2DMOE_F16;
  const hipError_t e = f16 ? launch_hidden_t<true>(A, sh.gated != 0, s) : launch_hidden_t<false>(A, sh.gated != 0, s);
  if (e != hipSuccess) return e;
  if (f16) launch_out_t<true>(A, L.nt16, (unsigned)(sh.d_model / 8), s);
  else launch_out_t<false>(A, L.nt16, (unsigned)(sh.d_model / 8), s);
  return hipGetLastError();
}

// The whole layer for at most 16 tokens in three launches: hidden activations of every expert + first router layer (one
// launch: neither waits for the other), second router layer (norms), output kernel with the selection inside.
bool mfma_decode_layer_supported(const d2dmoe_shape& sh) {
  return mfma_decode_supported(sh) && sh.n_tokens >= 1 && sh.n_tokens <= DC_MAX_TOKENS && sh.n_experts % 32 == 0 &&
         sh.n_experts <= DO_WAVES * 64 && sh.router_width > 0 && linear_skinny_supported(sh.n_tokens, sh.d_model, sh.dtype) &&
         linear_skinny_supported(sh.n_tokens, sh.router_width, sh.dtype);
}

hipError_t launch_mfma_decode_layer(const d2dmoe_shape& sh, const void* x, const void* router_w1, const void* router_w2,
                                    float thr_scale, const void* packed_section, const void* last_bias, void* router_hidden,
                                    void* norms, void* routing, int32_t* counts, void* out, void* workspace, hipStream_t s) {
  const DecodeLayout L = decode_layout(sh);
  const char* pk = (const char*)packed_section;
  DecodeArgs A;
  A.x = (const bf16_t*)x; A.routing = nullptr; A.wgu = (const bf16x8*)(pk + L.gu_off);
  A.wd = (const bf16x8*)(pk + L.d_off); A.bias = (const bf16_t*)(pk + L.b_off);
  A.hfrag = (bf16x8*)workspace; A.active = nullptr;
  A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out;
  A.N = (int)sh.n_tokens; A.D = sh.d_model; A.E = sh.n_experts; A.nt16 = L.nt16; A.act = sh.activation;
  A.add_residual = sh.add_residual;
  A.fused = 1; A.rw1 = (const bf16_t*)router_w1; A.rhidden = (bf16_t*)router_hidden; A.rwidth = sh.router_width;
  A.ract = sh.router_activation; A.norms = (const bf16_t*)norms; A.routing_out = (bf16_t*)routing; A.counts = counts;
  A.thr_scale = thr_scale;
  const bool f16 = sh.dtype == D2DMOE_F16;
  hipError_t e = f16 ? launch_hidden_t<true>(A, sh.gated != 0, s) : launch_hidden_t<false>(A, sh.gated != 0, s);
  if (e != hipSuccess) return e;
  e = launch_linear_skinny(router_hidden, router_w2, norms, (int)sh.n_tokens, sh.router_width, sh.n_experts,
                           sh.router_output_activation, s, sh.dtype);
  if (e != hipSuccess) return e;
  if (f16) launch_out_t<true>(A, L.nt16, (unsigned)(sh.d_model / 8), s);
  else launch_out_t<false>(A, L.nt16, (unsigned)(sh.d_model / 8), s);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Skinny Linear for <= 16 rows: C[N, Nout] = round(act(round(A[N,K] . B[Nout,K]^T))), bf16.
// Both operands are read straight from their row-major layouts (K contiguous in each): a workgroup owns 16 output features
// (4 where K is long and the features few, so that more than a handful of CUs pull on the weights), its 4 or 16 waves
// share K; partial tiles are summed through LDS in wave order.  Used for the router layers at small N.
// ---------------------------------------------------------------------------------------------------
template <int NW, int FPB, bool F16 = false>
__global__ __launch_bounds__(NW * 64) void linear_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
                                                               bf16_t* __restrict__ C, int N, int K, int Nout, int act) {
  __shared__ float part[NW][4][64];
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int gq = lane >> 4, c16 = lane & 15;
  const int f0 = blockIdx.x * FPB;                // first output feature of this workgroup
  const int KQ = K / NW;                          // per wave, a multiple of 32
  // FPB < 16: the rows of the 16-row tile past the workgroup's features repeat them (no extra traffic) and are dropped
  const int fr = f0 + (c16 & (FPB - 1));
  const int frow = (fr < Nout) ? fr : (Nout - 1);
  const int trow = (c16 < N) ? c16 : (N - 1);
  const bf16x8* bp = (const bf16x8*)(B + (int64_t)frow * K + w * KQ) + gq;
  const bf16x8* ap = (const bf16x8*)(A + (int64_t)trow * K + w * KQ) + gq;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int ks0 = 0; ks0 < KQ / 32; ks0 += 4) {   // four K steps requested together, then multiplied
    bf16x8 bv[4], av[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int ks = (ks0 + u < KQ / 32) ? (ks0 + u) : ks0;
      bv[u] = bp[ks * 4];
      av[u] = ap[ks * 4];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (ks0 + u < KQ / 32) acc = mfma_16x16x32<F16>(bv[u], av[u], acc);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) part[w][r][lane] = acc[r];
  __syncthreads();
  if (w == 0) {
    // C layout: lane holds token (column) c16, features 4 gq + r
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = part[0][r][lane];
#pragma unroll
      for (int ww = 1; ww < NW; ++ww) v += part[ww][r][lane];
      const int f = f0 + 4 * gq + r;
      if (c16 < N && f < Nout && 4 * gq + r < FPB) {
        const float vr = round16<F16>(v);
        C[(int64_t)c16 * Nout + f] = enc16<F16>(apply_act(act, vr));
      }
    }
  }
}

bool linear_skinny_supported(int64_t N, int K, int dtype) {
  return (dtype == D2DMOE_BF16 || dtype == D2DMOE_F16) && N >= 1 && N <= 16 && K % 128 == 0;
}

template <bool F16>
static void launch_linear_skinny_t(const void* A, const void* B, void* C, int N, int K, int Nout, int act, hipStream_t s) {
  if (K % 512 == 0 && K >= 1024) {   // long rows: 16 waves share K so that each requests its part in one go
    if (Nout <= 1024)
      hipLaunchKernelGGL((linear_skinny_kernel<16, 4, F16>), dim3((Nout + 3) / 4), dim3(1024), 0, s, (const bf16_t*)A,
                         (const bf16_t*)B, (bf16_t*)C, N, K, Nout, act);
    else
      hipLaunchKernelGGL((linear_skinny_kernel<16, 16, F16>), dim3((Nout + 15) / 16), dim3(1024), 0, s, (const bf16_t*)A,
                         (const bf16_t*)B, (bf16_t*)C, N, K, Nout, act);
  } else {
    hipLaunchKernelGGL((linear_skinny_kernel<4, 16, F16>), dim3((Nout + 15) / 16), dim3(256), 0, s, (const bf16_t*)A,
                       (const bf16_t*)B, (bf16_t*)C, N, K, Nout, act);
  }
}

hipError_t launch_linear_skinny(const void* A, const void* B, void* C, int N, int K, int Nout, int act, hipStream_t s, int dtype) {
  if (dtype == D2DMOE_F16) launch_linear_skinny_t<true>(A, B, C, N, K, Nout, act, s);
  else launch_linear_skinny_t<false>(A, B, C, N, K, Nout, act, s);
  return hipGetLastError();
}

}  // namespace d2dmoe
