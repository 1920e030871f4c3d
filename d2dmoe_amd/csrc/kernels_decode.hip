// Small-batch ("decode") bf16 MFMA path: at most 16 tokens, so the layer is bound by streaming the weights of the
// routed experts once.  One workgroup per expert pulls that expert's packed gate/up weights through
// v_mfma_f32_16x16x32_bf16 with all tokens resident in LDS and leaves the hidden activations (256 KB for 256 experts
// of 32 neurons) in memory; a second kernel owns 32 output columns and a range of experts per workgroup, requests that
// range's down-projection weights in one go, and sums the routed experts in ascending order (workgroups that share a
// column block add their partial sums in range order).  Also here: a skinny Linear kernel (router layers for <= 16
// tokens) that needs no packing.
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

constexpr int DO_WAVES = 8;
constexpr int DO_COLS = 32;          // output columns per workgroup of the output kernel
constexpr int DO_MAX_SPLIT = 16;     // expert ranges per column block at most

// Expert ranges per column block of the output kernel.  A wave keeps the down-projection fragments of all its experts in
// registers (KS2 * 12 registers per expert, 16 / KS2 experts at most), so a workgroup of 8 waves covers at most
// 128 / KS2 experts; beyond that, and while the grid would leave CUs without a workgroup, the experts are cut into more
// ranges.
static int decode_split(const d2dmoe_shape& sh) {
  const int ks2 = decode_layout(sh).nt16 / 2;
  const int per_wg = DO_WAVES * (16 / ks2);
  int q = (sh.n_experts + per_wg - 1) / per_wg;
  const int col_blocks = sh.d_model / DO_COLS;
  const int fill = (device_cu_count() + col_blocks - 1) / col_blocks;
  if (fill > q) q = fill;
  const int q_max = (sh.n_experts + DO_WAVES - 1) / DO_WAVES;   // at least one expert per wave
  if (q > q_max) q = q_max;
  if (q > DO_MAX_SPLIT) q = DO_MAX_SPLIT;
  return q < 1 ? 1 : q;
}

struct DecodeWorkspace { size_t hfrag, active, partial, tickets, total; };

static DecodeWorkspace decode_workspace(const d2dmoe_shape& sh) {
  DecodeWorkspace W;
  auto up = [](size_t v) { return (v + 255) / 256 * 256; };
  size_t off = 0;
  W.hfrag = off;   off += up((size_t)sh.n_experts * decode_layout(sh).edp * DC_MAX_TOKENS * 2);   // hidden fragments
  W.active = off;  off += up((size_t)sh.n_experts * 4);                                           // "some token routes here"
  // float32 partial sums [column block][range][16 tokens x 32 columns], sized for the largest split
  W.partial = off; off += up((size_t)(sh.d_model / DO_COLS) * DO_MAX_SPLIT * DC_MAX_TOKENS * DO_COLS * 4);
  W.tickets = off; off += up((size_t)(sh.d_model / DO_COLS) * 4);                                 // arrivals per column block
  W.total = off;
  return W;
}

size_t mfma_decode_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_decode_supported(sh)) return 0;
  return decode_workspace(sh).total;
}

// ---------------------------------------------------------------------------------------------------
// Packing.  KS = D/32 K steps, EdP padded neurons, NB = EdP/32 neuron blocks, NM = 2 if gated else 1.  Every workgroup of
// the two kernels below reads ONE contiguous stream.
//   gate(/up) stream [E][block NB][kstep KS][matrix NM][tile 2][lane 64][8]:
//                    neuron j = block*32 + tile*16 + c, d = kstep*32 + 8 gq + i                          w[e][d][j]
//   down^T stream    [column block D/32][E][kstep2 NB][column tile 2][lane 64][8]:  column = cb*32 + tile*16 + c,
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
  const int64_t n_d = (int64_t)(D / 32) * E * NB * 2 * 64;
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
    const int lane = (int)(q % 64); q /= 64;
    const int tile = (int)(q % 2); q /= 2;
    const int ks2 = (int)(q % NB); q /= NB;
    const int e = (int)(q % E);
    const int cb = (int)(q / E);
    const int gq = lane / 16;
    const int col = cb * 32 + tile * 16 + lane % 16;
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
// decode_out_kernel: workgroup = (block of 32 output columns, range of experts), 8 waves, two waves per SIMD.
//   Wave w owns a run of consecutive experts of the range.  It first requests the down-projection fragments of ALL of them
//   (nothing it has to compute decides that), then -- whole layer only -- works out the second router layer and the
//   selection while those loads are in flight, then requests the hidden fragments of its experts and chains
//   OUT^T += W2[e]^T . H[e]^T over them in ascending order in two float32 accumulators (one per tile of 16 columns).  The 8
//   partial tiles are added in wave order.  Ranges of one column block (when the experts are cut into several, so that
//   the grid covers the machine) leave their sums in the workspace; the last of them to arrive, found by an arrival
//   counter, adds them in range order.  Then last_bias, the residual, one rounding.  The summation order depends on the
//   routing and the launch shape only, never on timing.
// ---------------------------------------------------------------------------------------------------
struct DecodeArgs {
  const bf16_t* x; const bf16_t* routing; const bf16x8* wgu; const bf16x8* wd; const bf16_t* bias;
  bf16x8* hfrag; int* active; const bf16_t* last_bias; bf16_t* out; int N; int D; int E; int nt16; int act; int add_residual;
  // Whole layer in three launches (fused != 0): the hidden kernel computes every expert (it does not wait for the routing)
  // and its extra workgroups compute the first router layer; the output kernel derives the routing from the norms itself.
  int fused;
  const bf16_t* rw1; bf16_t* rhidden; int rwidth; int ract;     // first router layer: [rwidth, D] -> rhidden [N, rwidth]
  bf16_t* norms; bf16_t* routing_out; int32_t* counts; float thr_scale;
  const bf16_t* rw2; int roact;           // second router layer [E, rwidth], output activation (computed by the output kernel)
  float* partial; int* tickets; int split;   // output kernel: expert ranges per column block, their sums and arrival counters
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
  // the output kernel's arrival counters start at zero (it runs after this grid)
  if (blockIdx.x == gridDim.x - 1 && A.split > 1)
    for (int i = threadIdx.x; i < D / DO_COLS; i += 256) A.tickets[i] = 0;
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

// Second router layer for NT 16-feature tiles ft[0..NT), by one wave, with the bits of linear_skinny_kernel: K is cut into
// the same parts (16 where K is long, else 4), each accumulated on its own in K order, the parts summed in order, the sum
// rounded to the storage type before the activation.  nb[i][r]: the lane's norms of tile i (token c16, features
// ft[i]*16 + 4 gq + r) as storage bits.
// KQS > 0 (K = 128 * KQS, K steps of 32 per part): every operand is requested by router_l2_request before anything else
// of the kernel, so that these loads do not queue up behind the weight stream (a wave's loads return in order).
template <int NT, int KQS>
struct RouterL2Operands { bf16x8 av[KQS > 0 ? 4 * KQS : 1], bv[NT][KQS > 0 ? 4 * KQS : 1]; };

template <int NT, int KQS>
__device__ __forceinline__ void router_l2_request(const DecodeArgs& A, const int (&ft)[NT], int lane, RouterL2Operands<NT, KQS>& R) {
  if constexpr (KQS > 0) {
    const int gq = lane >> 4, c16 = lane & 15;
    const int K = A.rwidth;
    const int trow = (c16 < A.N) ? c16 : (A.N - 1);
    const bf16x8* ap = (const bf16x8*)(A.rhidden + (int64_t)trow * K) + gq;
#pragma unroll
    for (int ks = 0; ks < 4 * KQS; ++ks) R.av[ks] = ap[ks * 4];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const bf16x8* bp = (const bf16x8*)(A.rw2 + (int64_t)(ft[i] * 16 + c16) * K) + gq;
#pragma unroll
      for (int ks = 0; ks < 4 * KQS; ++ks) R.bv[i][ks] = bp[ks * 4];
    }
  }
}

template <bool F16, int NT, int KQS>
__device__ __forceinline__ void router_l2_finish(const DecodeArgs& A, const int (&ft)[NT], int lane, const RouterL2Operands<NT, KQS>& R,
                                                 uint16_t (&nb)[NT][4]) {
  float v[NT][4];
  if constexpr (KQS > 0) {
#pragma unroll
    for (int i = 0; i < NT; ++i) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < KQS; ++k) acc = mfma_16x16x32<F16>(R.bv[i][p * KQS + k], R.av[p * KQS + k], acc);
#pragma unroll
        for (int r = 0; r < 4; ++r) v[i][r] = (p == 0) ? acc[r] : v[i][r] + acc[r];
      }
    }
  } else {
    const int gq = lane >> 4, c16 = lane & 15;
    const int K = A.rwidth;
    const int trow = (c16 < A.N) ? c16 : (A.N - 1);
    const bf16x8* ap = (const bf16x8*)(A.rhidden + (int64_t)trow * K) + gq;
    const int P = (K % 512 == 0 && K >= 1024) ? 16 : 4;
    const int KQ = K / P;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const bf16x8* bp = (const bf16x8*)(A.rw2 + (int64_t)(ft[i] * 16 + c16) * K) + gq;
      for (int p = 0; p < P; ++p) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int ks = 0; ks < KQ / 32; ++ks) acc = mfma_16x16x32<F16>(bp[(p * (KQ / 32) + ks) * 4], ap[(p * (KQ / 32) + ks) * 4], acc);
#pragma unroll
        for (int r = 0; r < 4; ++r) v[i][r] = (p == 0) ? acc[r] : v[i][r] + acc[r];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) nb[i][r] = enc16<F16>(apply_act(A.roact, round16<F16>(v[i][r])));
}

// Workgroup = (column block cb, expert range q): blockIdx.x = cb * split + q.  KS2 = 32-neuron K steps per expert.
// KQS: see router_l2_request (whole layer with a router of width 128 * KQS; 0 otherwise).
template <int KS2, bool F16 = false, int KQS = 0>
__global__ __launch_bounds__(DO_WAVES * 64) void decode_out_kernel(const DecodeArgs A) {
  constexpr int ME = 16 / KS2;                 // experts a wave keeps in registers at most
  __shared__ float part[DO_WAVES][2][4][64];
  __shared__ float s_thr[16];                  // fused: the tokens' thresholds
  __shared__ unsigned short s_bits[DO_WAVES * 64];   // fused: per expert, bit t = token t routes to it
  __shared__ bf16_t s_norms[DC_MAX_TOKENS][DO_WAVES * 64 + 8];   // fused: the norms tile
  __shared__ int s_last;
  const int D = A.D, N = A.N, E = A.E;
  const int t = threadIdx.x, lane = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);   // uniform: the branches on a wave's experts are scalar
  const int gq = lane >> 4, c16 = lane & 15;
  const int Q = A.split;
  const int cb = (int)blockIdx.x / Q, q = (int)blockIdx.x % Q;
  const int EPG = (E + Q - 1) / Q;                              // experts per range
  const int EPW = (EPG + DO_WAVES - 1) / DO_WAVES;              // ... per wave (<= ME: the launcher's choice of Q)
  const int g_lo = q * EPG, g_hi = (g_lo + EPG < E) ? (g_lo + EPG) : E;
  const int e_lo = g_lo + w * EPW;
  const int e_hi = (e_lo + EPW < g_hi) ? (e_lo + EPW) : g_hi;   // may be <= e_lo: a wave without experts

  // ---- 0. whole layer: the operands of this wave's first two tiles of the second router layer, ahead of everything
  const int E16 = E / 16;
  int ft_first[2] = {w < E16 ? w : 0, (w + DO_WAVES < E16) ? (w + DO_WAVES) : (w < E16 ? w : 0)};
  RouterL2Operands<2, KQS> rl2;
  if (A.fused) router_l2_request<2, KQS>(A, ft_first, lane, rl2);

  // ---- 1. the down-projection fragments of every expert of this wave (not fused: of those some token routes to; the
  // flags of the wave's experts come in with one load and a ballot, so that the branches below are scalar and no load
  // waits for another)
  bf16x8 wa[ME][KS2][2];
  unsigned umask;                              // bit j: expert e_lo + j is in use
  {
    const int e = e_lo + (lane < ME ? lane : 0);
    const bool mine = lane < ME && lane < EPW && e < e_hi;
    const int flag = (A.fused || !mine) ? 1 : A.active[e];
    umask = (unsigned)__ballot(mine && flag != 0);
  }
  const bf16x8* wdf = A.wd + (int64_t)cb * E * KS2 * 2 * 64 + lane;
  const bf16x8 zero8 = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
  auto request_weights = [&](auto j_c) __attribute__((always_inline)) {
    constexpr int j = decltype(j_c)::value;
    if constexpr (KQS > 0) {
      // whole layer: every expert of the wave, without a branch (the compiler can then count the loads that follow the
      // router's and wait for those alone); a slot past the wave's experts repeats a valid expert and is cleared later
      const int e = (e_lo + j < E) ? (e_lo + j) : (E - 1);
#pragma unroll
      for (int k2 = 0; k2 < KS2; ++k2)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) wa[j][k2][ct] = wdf[(((int64_t)e * KS2 + k2) * 2 + ct) * 64];
    } else if ((umask >> j) & 1u) {
#pragma unroll
      for (int k2 = 0; k2 < KS2; ++k2)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) wa[j][k2][ct] = wdf[(((int64_t)(e_lo + j) * KS2 + k2) * 2 + ct) * 64];
    } else {
#pragma unroll
      for (int k2 = 0; k2 < KS2; ++k2)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) wa[j][k2][ct] = zero8;
    }
  };
  // (whole layer with the router operands in registers: the last quarter of the experts is requested once those
  // registers are free again, or the kernel spills -- and a reload from scratch would queue up behind the weight stream)
  constexpr int ME_FIRST = (KQS > 0) ? (ME - ME / 4) : ME;
  static_for<0, ME_FIRST>(request_weights);
  __builtin_amdgcn_sched_barrier(0);

  if (A.fused) {
    // ---- 2. second router layer (every workgroup for itself: rwidth * E * 2 bytes out of L2) and the dynamic-k selection
    // (moefication.py:80-85).  Wave w takes the feature tiles w, w + 8, ...; wave 0 then takes the maximum of every
    // token's row, and a thread per expert compares its column with the thresholds.  Same arithmetic as select_kernel:
    // m NaN-propagating, thr = round(m * thr_scale), on = norm >= thr.
    // (two tiles at a time; the tile index of a wave without a second tile repeats its first: same values, same place)
    for (int ft0 = w; ft0 < E16; ft0 += 2 * DO_WAVES) {
      const int ft[2] = {ft0, (ft0 + DO_WAVES < E16) ? (ft0 + DO_WAVES) : ft0};
      uint16_t nb[2][4];
      if (ft0 == w) {
        router_l2_finish<F16, 2, KQS>(A, ft, lane, rl2, nb);          // requested at the top
      } else {
        RouterL2Operands<2, 0> none;
        router_l2_finish<F16, 2, 0>(A, ft, lane, none, nb);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) s_norms[c16][ft[i] * 16 + 4 * gq + r] = nb[i][r];
      }
    }
    static_for<ME_FIRST, ME>(request_weights);
    __builtin_amdgcn_sched_barrier(0);
    // (barriers of this phase order LDS traffic only: __syncthreads would wait for the weight loads in flight)
    lds_barrier();
    if (w == 0) {
      float m = -INFINITY;
      for (int e8 = gq * 8; e8 < E; e8 += 32) {          // E is a multiple of 32 here
        const u32x4 v = *(const u32x4*)(&s_norms[c16][e8]);
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
    lds_barrier();
    if (t < E) {
      unsigned bits = 0u;
#pragma unroll
      for (int tk = 0; tk < DC_MAX_TOKENS; ++tk) bits |= ((tk < N && dec16<F16>(s_norms[tk][t]) >= s_thr[tk]) ? 1u : 0u) << tk;
      s_bits[t] = (unsigned short)bits;
      // The layer's other outputs as 2 N + 1 jobs dealt round-robin to the workgroups, so that none is held up: job
      // j < N is row j of the routing tensor, job N + j row j of the norms, job 2 N the counts.
      for (int j = (int)blockIdx.x; j <= 2 * N; j += (int)gridDim.x) {
        if (j < N) A.routing_out[(int64_t)j * E + t] = ((bits >> j) & 1u) ? (bf16_t)(F16 ? 0x3c00 : 0x3f80) : (bf16_t)0;
        else if (j < 2 * N) A.norms[(int64_t)(j - N) * E + t] = s_norms[j - N][t];
        else if (A.counts != nullptr) A.counts[t] = __popc(bits);
      }
    }
    lds_barrier();
  }

  // ---- 3. hidden fragments of all the wave's experts in one go (an expert out of use: some valid fragment, multiplied by
  // zero weights or cleared below), then the products in ascending expert order, without a branch
  const bf16x8* hf = A.hfrag + lane;
  bf16x8 hb[ME][KS2];
#pragma unroll
  for (int j = 0; j < ME; ++j) {
    const int e = (e_lo + j < E) ? (e_lo + j) : (E - 1);
#pragma unroll
    for (int k2 = 0; k2 < KS2; ++k2) hb[j][k2] = hf[((int64_t)e * KS2 + k2) * 64];
  }
  f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
  for (int j = 0; j < ME; ++j) {
    // the columns of tokens that do not route here are cleared (fused: the hidden fragment holds every token; not fused:
    // an expert out of use may hold anything)
    bool keep = ((umask >> j) & 1u) != 0u;
    if (A.fused) keep = keep && (((s_bits[(e_lo + j < E) ? (e_lo + j) : (E - 1)] >> c16) & 1u) != 0u);
#pragma unroll
    for (int k2 = 0; k2 < KS2; ++k2) {
      u32x4 bm = __builtin_bit_cast(u32x4, hb[j][k2]);
      bm.x = keep ? bm.x : 0u; bm.y = keep ? bm.y : 0u; bm.z = keep ? bm.z : 0u; bm.w = keep ? bm.w : 0u;
      const bf16x8 bv = __builtin_bit_cast(bf16x8, bm);
      acc[0] = mfma_16x16x32<F16>(wa[j][k2][0], bv, acc[0]);
      acc[1] = mfma_16x16x32<F16>(wa[j][k2][1], bv, acc[1]);
    }
  }
#pragma unroll
  for (int ct = 0; ct < 2; ++ct)
#pragma unroll
    for (int r = 0; r < 4; ++r) part[w][ct][r][lane] = acc[ct][r];
  lds_barrier();

  // ---- 4. waves in order; thread (ct, lane) of the first 128 ends with token c16 and 4 consecutive columns
  const int ct = (t >> 6) & 1;
  float o[4] = {0.f, 0.f, 0.f, 0.f};
  if (t < 128) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sacc = part[0][ct][r][lane];
#pragma unroll
      for (int ww = 1; ww < DO_WAVES; ++ww) sacc += part[ww][ct][r][lane];
      o[r] = sacc;
    }
  }
  if (Q > 1) {
    // Leave this range's sums and count the arrival; the last range of the column block to arrive adds all of them in range
    // order.  Sums and counter are written and read with device-scope atomic accesses only: such a store is written
    // through to the memory side (the ranges ran on other CUs, maybe other XCDs, whose L2 caches do not snoop each other),
    // such a load is not served from a stale line, and the barrier ahead of the counter update has waited for every
    // thread's stores to be acknowledged.  No release / acquire fences: a fence in every wave (an L2 write-back and
    // invalidation each) made this kernel four times slower, and even the one pair hung on the counter update cost 2.8 us
    // of the kernel's 15.
    float* mine = A.partial + ((int64_t)cb * Q + q) * (DC_MAX_TOKENS * DO_COLS);
    if (t < 128) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        __hip_atomic_store(mine + t * 4 + r, o[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (t == 0) {
      const int arrived = __hip_atomic_fetch_add(A.tickets + cb, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (arrived == Q - 1) ? 1 : 0;
    }
    __syncthreads();
    if (s_last == 0) return;
    if (t < 128) {
      const float* all = A.partial + (int64_t)cb * Q * (DC_MAX_TOKENS * DO_COLS);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float sacc = 0.f;
        for (int qq = 0; qq < Q; ++qq) {
          const float v = __hip_atomic_load(all + (int64_t)qq * (DC_MAX_TOKENS * DO_COLS) + t * 4 + r, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
          sacc = (qq == 0) ? v : sacc + v;
        }
        o[r] = sacc;
      }
    }
  }
  if (t < 128 && c16 < N) {
    // C layout (transposed product): lane holds token c16, rows 4 gq + r = columns cb*32 + ct*16 + 4 gq + r
    const int col = cb * DO_COLS + ct * 16 + 4 * gq;
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
template <bool F16, int KQS>
static void launch_out_q(const DecodeArgs& A, int nt16, unsigned grid, hipStream_t s) {
  if (nt16 == 2) hipLaunchKernelGGL((decode_out_kernel<1, F16, KQS>), dim3(grid), dim3(DO_WAVES * 64), 0, s, A);
  else if (nt16 == 4) hipLaunchKernelGGL((decode_out_kernel<2, F16, KQS>), dim3(grid), dim3(DO_WAVES * 64), 0, s, A);
  else hipLaunchKernelGGL((decode_out_kernel<4, F16, KQS>), dim3(grid), dim3(DO_WAVES * 64), 0, s, A);
}
template <bool F16>
static void launch_out_t(const DecodeArgs& A, int nt16, unsigned grid, hipStream_t s) {
  if (A.fused && A.rwidth == 256) launch_out_q<F16, 2>(A, nt16, grid, s);
  else if (A.fused && A.rwidth == 128) launch_out_q<F16, 1>(A, nt16, grid, s);
  else launch_out_q<F16, 0>(A, nt16, grid, s);
}

hipError_t launch_mfma_decode(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                              const void* last_bias, void* out, void* workspace, hipStream_t s) {
  const DecodeLayout L = decode_layout(sh);
  const char* pk = (const char*)packed_section;
  DecodeArgs A;
  A.x = (const bf16_t*)x; A.routing = (const bf16_t*)routing; A.wgu = (const bf16x8*)(pk + L.gu_off);
  A.wd = (const bf16x8*)(pk + L.d_off); A.bias = (const bf16_t*)(pk + L.b_off);
  A.hfrag = (bf16x8*)workspace;
  const DecodeWorkspace WS = decode_workspace(sh);
  A.active = (int*)((char*)workspace + WS.active);
  A.partial = (float*)((char*)workspace + WS.partial); A.tickets = (int*)((char*)workspace + WS.tickets);
  A.split = decode_split(sh); A.rw2 = nullptr; A.roact = 0;
  A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out;
  A.N = (int)sh.n_tokens; A.D = sh.d_model; A.E = sh.n_experts; A.nt16 = L.nt16; A.act = sh.activation;
  A.add_residual = sh.add_residual;
  A.fused = 0; A.rw1 = nullptr; A.rhidden = nullptr; A.rwidth = 0; A.ract = 0; A.norms = nullptr; A.routing_out = nullptr;
  A.counts = nullptr; A.thr_scale = 0.f;
  const bool f16 = sh.dtype == D2DMOE_F16;
  const hipError_t e = f16 ? launch_hidden_t<true>(A, sh.gated != 0, s) : launch_hidden_t<false>(A, sh.gated != 0, s);
  if (e != hipSuccess) return e;
  if (f16) launch_out_t<true>(A, L.nt16, (unsigned)(sh.d_model / DO_COLS * A.split), s);
  else launch_out_t<false>(A, L.nt16, (unsigned)(sh.d_model / DO_COLS * A.split), s);
  return hipGetLastError();
}

// The whole layer for at most 16 tokens in two launches: hidden activations of every expert + first router layer (one
// launch: neither waits for the other), then the output kernel, which requests its weights, works out the second router
// layer and the selection while they travel, and multiplies.
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
  const DecodeWorkspace WS = decode_workspace(sh);
  A.hfrag = (bf16x8*)workspace; A.active = nullptr;
  A.partial = (float*)((char*)workspace + WS.partial); A.tickets = (int*)((char*)workspace + WS.tickets);
  A.split = decode_split(sh); A.rw2 = (const bf16_t*)router_w2; A.roact = sh.router_output_activation;
  A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out;
  A.N = (int)sh.n_tokens; A.D = sh.d_model; A.E = sh.n_experts; A.nt16 = L.nt16; A.act = sh.activation;
  A.add_residual = sh.add_residual;
  A.fused = 1; A.rw1 = (const bf16_t*)router_w1; A.rhidden = (bf16_t*)router_hidden; A.rwidth = sh.router_width;
  A.ract = sh.router_activation; A.norms = (bf16_t*)norms; A.routing_out = (bf16_t*)routing; A.counts = counts;
  A.thr_scale = thr_scale;
  const bool f16 = sh.dtype == D2DMOE_F16;
  hipError_t e = f16 ? launch_hidden_t<true>(A, sh.gated != 0, s) : launch_hidden_t<false>(A, sh.gated != 0, s);
  if (e != hipSuccess) return e;
  if (f16) launch_out_t<true>(A, L.nt16, (unsigned)(sh.d_model / DO_COLS * A.split), s);
  else launch_out_t<false>(A, L.nt16, (unsigned)(sh.d_model / DO_COLS * A.split), s);
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
