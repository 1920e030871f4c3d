// Small-batch ("decode") bf16 MFMA path: at most 16 tokens, so the layer is bound by streaming the weights of the
// routed experts once.  One workgroup per expert pulls that expert's packed weights (gate/up and down projections)
// through v_mfma_f32_16x16x32_bf16 with all tokens resident in LDS; per-expert results are summed afterwards in
// ascending expert order.  Also here: a skinny Linear kernel (router layers for <= 16 tokens) that needs no packing.
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
  size_t g_off, u_off, d_off, b_off, total;   // gate (or w1), up, down^T fragments, bias (bf16, padded)
};

static DecodeLayout decode_layout(const d2dmoe_shape& sh) {
  DecodeLayout L;
  L.edp = (sh.expert_dim + 31) / 32 * 32;
  L.nt16 = L.edp / 16;
  const size_t mat = (size_t)sh.n_experts * L.edp * sh.d_model * 2;
  size_t off = 0;
  L.g_off = off; off += mat;
  L.u_off = off; if (sh.gated) off += mat;
  L.d_off = off; off += mat;
  L.b_off = off; off += (size_t)sh.n_experts * L.edp * 2;
  L.total = (off + 255) / 256 * 256;
  return L;
}

bool mfma_decode_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16) return false;
  if (sh.d_model % 256 != 0 || sh.d_model > 4096) return false;   // K quarters of whole 32-steps, column tiles in fours
  const int edp = (sh.expert_dim + 31) / 32 * 32;
  return edp == 32 || edp == 64 || edp == 128;
}

size_t mfma_decode_packed_bytes(const d2dmoe_shape& sh) { return mfma_decode_supported(sh) ? decode_layout(sh).total : 0; }

size_t mfma_decode_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_decode_supported(sh)) return 0;
  return (size_t)sh.n_experts * DC_MAX_TOKENS * sh.d_model * 2;   // per-expert result rows, bf16
}

// ---------------------------------------------------------------------------------------------------
// Packing.  KS = D/32 K steps, nt16 neuron tiles, EdP padded neurons.
//   gate / up fragments [E][kstep KS][nt16][lane][8]:  neuron j = t*16 + c, d = kstep*32 + 8 gq + i     w[e][d][j]
//   down^T fragments    [E][col-tile D/16][kstep2 EdP/32][lane][8]:  column = ct*16 + c,
//                       neuron j = ks2*32 + 16*(i/4) + 4 gq + (i%4)                                       w2[e][j][column]
//   bias                [E][EdP] bf16
// ---------------------------------------------------------------------------------------------------
__global__ void pack_decode_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ b1, const bf16_t* __restrict__ w2,
                                   const bf16_t* __restrict__ w_up, bf16_t* __restrict__ dg, bf16_t* __restrict__ du,
                                   bf16_t* __restrict__ dd, bf16_t* __restrict__ db, int D, int E, int Ed, int edp) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per_expert = (int64_t)edp * D / 8;   // 16-byte pieces per expert and matrix
  const int64_t n = (int64_t)E * per_expert;
  const int lane = (int)(p % 64);
  const int gq = lane / 16, c = lane % 16;
  const int nt16 = edp / 16;
  if (p < 2 * n) {   // gate, then up
    const bool is_up = p >= n;
    const int64_t pp = is_up ? p - n : p;
    if (is_up && w_up == nullptr) return;
    const bf16_t* src = is_up ? w_up : w1;
    bf16_t* dst = is_up ? du : dg;
    const int e = (int)(pp / per_expert);
    const int64_t q = (pp % per_expert) / 64;
    const int t = (int)(q % nt16), ks = (int)(q / nt16);
    const int j = t * 16 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 32 + 8 * gq + i;
      dst[pp * 8 + i] = (j < Ed) ? src[((int64_t)e * D + d) * Ed + j] : (bf16_t)0;
    }
  } else if (p < 3 * n) {
    const int64_t pp = p - 2 * n;
    const int e = (int)(pp / per_expert);
    const int64_t q = (pp % per_expert) / 64;
    const int nks2 = edp / 32;
    const int ks2 = (int)(q % nks2), ct = (int)(q / nks2);
    const int col = ct * 16 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = ks2 * 32 + 16 * (i / 4) + 4 * gq + (i % 4);
      dd[pp * 8 + i] = (j < Ed) ? w2[((int64_t)e * Ed + j) * D + col] : (bf16_t)0;
    }
  } else if (p < 3 * n + (int64_t)E * edp) {
    const int64_t pp = p - 3 * n;
    const int e = (int)(pp / edp), j = (int)(pp % edp);
    db[pp] = (j < Ed && b1 != nullptr) ? b1[(int64_t)e * Ed + j] : (bf16_t)0;
  }
}

hipError_t launch_decode_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                              void* packed_section, hipStream_t s) {
  const DecodeLayout L = decode_layout(sh);
  char* base = (char*)packed_section;
  const int64_t n = 3 * (int64_t)sh.n_experts * L.edp * sh.d_model / 8 + (int64_t)sh.n_experts * L.edp;
  hipLaunchKernelGGL(pack_decode_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)w1, (const bf16_t*)b1,
                     (const bf16_t*)w2, (const bf16_t*)w_up, (bf16_t*)(base + L.g_off), (bf16_t*)(base + L.u_off),
                     (bf16_t*)(base + L.d_off), (bf16_t*)(base + L.b_off), sh.d_model, sh.n_experts, sh.expert_dim, L.edp);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Decode experts kernel: workgroup = expert, 4 waves.
//   stage   x [N <= 16, D] as B fragments in LDS (rows beyond N are zero); leave at once if no token routes here
//   GEMM1   wave w: its quarter of K for all neuron tiles, gate and (if gated) up; partial tiles summed through LDS
//           in wave order
//   hidden  gated: act(g) * u, else act(g + b1); times the routing weight; rounded to bf16 -> B fragments
//   GEMM2   wave w: D/4 output columns, OUT^T = W2^T . H^T; the lane's token row of y[e] gets 8-byte stores
// ---------------------------------------------------------------------------------------------------
struct DecodeArgs {
  const bf16_t* x; const bf16_t* routing; const bf16x8* wg; const bf16x8* wu; const bf16x8* wd; const bf16_t* bias;
  bf16_t* y; int N; int D; int E; int act; int gated;
};

template <int NT16, bool GATED, int U1, int U2>
__global__ __launch_bounds__(256) void decode_experts_kernel(const DecodeArgs A) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int D = A.D, N = A.N, E = A.E;
  const int KS = D / 32;          // K steps of GEMM1
  const int KQ = KS / 4;          // per wave
  constexpr int NM = GATED ? 2 : 1;
  constexpr int KS2 = NT16 / 2;   // K steps of GEMM2
  bf16x8* xs = (bf16x8*)smem_raw;                                   // [KS][64]
  float* part = (float*)(xs + (size_t)KS * 64);                     // [4][NM*NT16*4][64]
  int* s_any = (int*)(part + 4 * NM * NT16 * 4 * 64);
  const int e = blockIdx.x;
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int gq = lane >> 4, c16 = lane & 15;
  if (t == 0) *s_any = 0;
  __syncthreads();
  if (t < N && (A.routing[(int64_t)t * E + e] & 0x7fff) != 0) *s_any = 1;
  // x tile -> B fragments: fragment (ks, lane) = x[token c16][ks*32 + 8 gq .. +7]
  for (int p = t; p < KS * 64; p += 256) {
    const int ks = p >> 6, l = p & 63;
    const int tok = l & 15, g4 = l >> 4;
    uint4 v = {0u, 0u, 0u, 0u};
    if (tok < N) v = *(const uint4*)(A.x + (int64_t)tok * D + ks * 32 + 8 * g4);
    ((uint4*)xs)[p] = v;
  }
  __syncthreads();
  if (*s_any == 0) return;   // nobody routes to this expert: its rows of y are never read

  // ---- GEMM1, this wave's quarter of K
  f32x4 acc1[NM][NT16];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int a = 0; a < NT16; ++a) acc1[m][a] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int64_t mat_frags = (int64_t)KS * NT16 * 64;
  const bf16x8* wgf = A.wg + (int64_t)e * mat_frags + (int64_t)w * KQ * NT16 * 64 + lane;
  const bf16x8* wuf = GATED ? (A.wu + (int64_t)e * mat_frags + (int64_t)w * KQ * NT16 * 64 + lane) : nullptr;
  for (int ks0 = 0; ks0 < KQ; ks0 += U1) {   // U1 K steps per trip: their weight fragments are in flight together
    bf16x8 b[U1], ag[U1][NT16], au[U1][NT16];
#pragma unroll
    for (int u = 0; u < U1; ++u) {
      b[u] = xs[(w * KQ + ks0 + u) * 64 + lane];
#pragma unroll
      for (int a = 0; a < NT16; ++a) {
        ag[u][a] = wgf[((ks0 + u) * NT16 + a) * 64];
        if (GATED) au[u][a] = wuf[((ks0 + u) * NT16 + a) * 64];
      }
    }
#pragma unroll
    for (int u = 0; u < U1; ++u)
#pragma unroll
      for (int a = 0; a < NT16; ++a) {
        acc1[0][a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ag[u][a], b[u], acc1[0][a], 0, 0, 0);
        if (GATED) acc1[NM - 1][a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(au[u][a], b[u], acc1[NM - 1][a], 0, 0, 0);
      }
  }
  // W2^T fragments of this wave's columns: the first batch is requested before the reduction below
  const int CTW = D / 64;   // 16-column tiles per wave
  const bf16x8* wdf = A.wd + ((int64_t)e * (D / 16) + (int64_t)w * CTW) * KS2 * 64 + lane;
  bf16x8 a2[U2][KS2];
#pragma unroll
  for (int j = 0; j < U2; ++j)
#pragma unroll
    for (int k2 = 0; k2 < KS2; ++k2) a2[j][k2] = wdf[(j * KS2 + k2) * 64];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int a = 0; a < NT16; ++a)
#pragma unroll
      for (int r = 0; r < 4; ++r) part[((w * NM + m) * NT16 * 4 + a * 4 + r) * 64 + lane] = acc1[m][a][r];
  __syncthreads();
  // ---- hidden activations -> B fragments of GEMM2
  const float rw = (c16 < N) ? bf16_to_f32(A.routing[(int64_t)c16 * E + e]) : 0.f;
  const bf16_t* bias_e = A.bias + (int64_t)e * NT16 * 16;
  bf16x8 hb[KS2];
#pragma unroll
  for (int k2 = 0; k2 < KS2; ++k2) {
    float hv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int a = 2 * k2 + (i >> 2), r = i & 3;
      float gsum = 0.f, usum = 0.f;
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) {
        gsum += part[((ww * NM + 0) * NT16 * 4 + a * 4 + r) * 64 + lane];
        if (GATED) usum += part[((ww * NM + NM - 1) * NT16 * 4 + a * 4 + r) * 64 + lane];
      }
      float v;
      if (GATED) {
        v = apply_act(A.act, gsum) * usum;
      } else {
        v = apply_act(A.act, gsum + bf16_to_f32(bias_e[a * 16 + 4 * gq + r]));
      }
      hv[i] = v * rw;
    }
    uint4 pk;
    pk.x = pack2_bf16(hv[0], hv[1]); pk.y = pack2_bf16(hv[2], hv[3]);
    pk.z = pack2_bf16(hv[4], hv[5]); pk.w = pack2_bf16(hv[6], hv[7]);
    __builtin_memcpy(&hb[k2], &pk, 16);
  }
  // ---- GEMM2 (transposed), U2 column tiles at a time, double-buffered in registers
  bf16_t* yrow = A.y + ((int64_t)e * DC_MAX_TOKENS + c16) * D + (int64_t)w * (D / 4) + 4 * gq;
  for (int ct0 = 0; ct0 < CTW; ct0 += U2) {
    bf16x8 a[U2][KS2];
#pragma unroll
    for (int j = 0; j < U2; ++j)
#pragma unroll
      for (int k2 = 0; k2 < KS2; ++k2) {
        a[j][k2] = a2[j][k2];
        // request the next batch while this one is multiplied (the last trip re-reads its own batch: in bounds)
        const int ctn = (ct0 + U2 < CTW) ? (ct0 + U2) : ct0;
        a2[j][k2] = wdf[((ctn + j) * KS2 + k2) * 64];
      }
#pragma unroll
    for (int j = 0; j < U2; ++j) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k2 = 0; k2 < KS2; ++k2) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j][k2], hb[k2], acc, 0, 0, 0);
      if (c16 < N) {
        uint2 o;
        o.x = pack2_bf16(acc[0], acc[1]);
        o.y = pack2_bf16(acc[2], acc[3]);
        *(uint2*)(yrow + (ct0 + j) * 16) = o;
      }
    }
  }
}

// Combine for the decode path.  A workgroup owns one token and 128 output columns: 16 column pieces (8 columns, 16
// bytes) x 16 expert groups.  Thread (piece, group) adds its group's routed experts in ascending order; the 16 group
// sums are then added in ascending group order.  The summation order is fixed, so results are reproducible.
__global__ __launch_bounds__(256) void decode_combine_kernel(const bf16_t* __restrict__ y, const bf16_t* __restrict__ routing,
                                                             const bf16_t* __restrict__ x, const bf16_t* __restrict__ last_bias,
                                                             bf16_t* __restrict__ out, int N, int D, int E, int add_residual) {
  __shared__ float part[16][16][9];   // [group][piece][8 columns + pad]
  const int t = threadIdx.x;
  const int piece = t & 15, grp = t >> 4;
  const int blocks_per_token = D / 128;
  const int n = blockIdx.x / blocks_per_token;
  const int col = (blockIdx.x % blocks_per_token) * 128 + piece * 8;
  const int per = (E + 15) / 16;            // experts per group
  const int e_lo = grp * per, e_hi = (e_lo + per < E) ? (e_lo + per) : E;
  const bf16_t* rrow = routing + (int64_t)n * E;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  for (int e0 = e_lo; e0 < e_hi; e0 += 8) {
    uint4 v[8];
    bool on[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      on[j] = (e0 + j < e_hi) && ((rrow[e0 + j] & 0x7fff) != 0);
      v[j] = uint4{0u, 0u, 0u, 0u};
      if (on[j]) v[j] = *(const uint4*)(y + ((int64_t)(e0 + j) * DC_MAX_TOKENS + n) * D + col);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (on[j]) {
        const uint32_t wd[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += __uint_as_float((i & 1) ? (wd[i >> 1] & 0xffff0000u) : (wd[i >> 1] << 16));
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[grp][piece][i] = acc[i];
  __syncthreads();
  if (grp == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float s = part[0][piece][i];
      for (int gi = 1; gi < 16; ++gi) s += part[gi][piece][i];
      acc[i] = s;
    }
    if (last_bias != nullptr) {
      const uint4 v = *(const uint4*)(last_bias + col);
      const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += __uint_as_float((i & 1) ? (wd[i >> 1] & 0xffff0000u) : (wd[i >> 1] << 16));
    }
    if (add_residual) {
      const uint4 v = *(const uint4*)(x + (int64_t)n * D + col);
      const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += __uint_as_float((i & 1) ? (wd[i >> 1] & 0xffff0000u) : (wd[i >> 1] << 16));
    }
    uint4 o;
    o.x = pack2_bf16(acc[0], acc[1]); o.y = pack2_bf16(acc[2], acc[3]);
    o.z = pack2_bf16(acc[4], acc[5]); o.w = pack2_bf16(acc[6], acc[7]);
    *(uint4*)(out + (int64_t)n * D + col) = o;
  }
}

template <int NT16, bool GATED, int U1, int U2>
static hipError_t launch_decode_cfg(const DecodeArgs& A, size_t lds, hipStream_t s) {
  auto k = decode_experts_kernel<NT16, GATED, U1, U2>;
  hipError_t e = hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(k, dim3(A.E), dim3(256), lds, s, A);
  return hipGetLastError();
}

template <int NT16>
static hipError_t launch_decode_nt(const DecodeArgs& A, size_t lds, hipStream_t s) {
  // deeper batches when the per-wave trip counts divide: K steps per wave = D/128, column tiles per wave = D/64
  const bool deep = (A.D % 512 == 0);
  if (A.gated) {
    if (deep && NT16 <= 4) return launch_decode_cfg<NT16, true, 4, 8>(A, lds, s);
    return launch_decode_cfg<NT16, true, 2, 4>(A, lds, s);
  }
  if (deep && NT16 <= 4) return launch_decode_cfg<NT16, false, 4, 8>(A, lds, s);
  return launch_decode_cfg<NT16, false, 2, 4>(A, lds, s);
}

hipError_t launch_mfma_decode(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                              const void* last_bias, void* out, void* workspace, hipStream_t s) {
  const DecodeLayout L = decode_layout(sh);
  const char* pk = (const char*)packed_section;
  DecodeArgs A;
  A.x = (const bf16_t*)x; A.routing = (const bf16_t*)routing; A.wg = (const bf16x8*)(pk + L.g_off);
  A.wu = (const bf16x8*)(pk + L.u_off); A.wd = (const bf16x8*)(pk + L.d_off); A.bias = (const bf16_t*)(pk + L.b_off);
  A.y = (bf16_t*)workspace; A.N = (int)sh.n_tokens; A.D = sh.d_model; A.E = sh.n_experts; A.act = sh.activation;
  A.gated = sh.gated;
  const int nm = sh.gated ? 2 : 1;
  const size_t lds = (size_t)(sh.d_model / 32) * 64 * 16 + (size_t)4 * nm * L.nt16 * 4 * 64 * 4 + 16;
  hipError_t e;
  if (L.nt16 == 2) e = launch_decode_nt<2>(A, lds, s);
  else if (L.nt16 == 4) e = launch_decode_nt<4>(A, lds, s);
  else e = launch_decode_nt<8>(A, lds, s);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(decode_combine_kernel, dim3((unsigned)sh.n_tokens * (sh.d_model / 128)), dim3(256), 0, s, (const bf16_t*)workspace,
                     (const bf16_t*)routing, (const bf16_t*)x, (const bf16_t*)last_bias, (bf16_t*)out, (int)sh.n_tokens,
                     sh.d_model, sh.n_experts, sh.add_residual);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Skinny Linear for <= 16 rows: C[N, Nout] = round(act(round(A[N,K] . B[Nout,K]^T))), bf16.
// Both operands are read straight from their row-major layouts (K contiguous in each): a wave owns 16 output features
// and a quarter of K; partial tiles are summed through LDS in wave order.  Used for the router layers at small N.
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void linear_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
                                                            bf16_t* __restrict__ C, int N, int K, int Nout, int act) {
  __shared__ float part[4][4][64];
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int gq = lane >> 4, c16 = lane & 15;
  const int f0 = blockIdx.x * 16;                 // first output feature of this workgroup
  const int KQ = K / 4;                           // per wave, a multiple of 32
  const int frow = (f0 + c16 < Nout) ? (f0 + c16) : (Nout - 1);
  const int trow = (c16 < N) ? c16 : (N - 1);
  const bf16x8* bp = (const bf16x8*)(B + (int64_t)frow * K + w * KQ) + gq;
  const bf16x8* ap = (const bf16x8*)(A + (int64_t)trow * K + w * KQ) + gq;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int ks = 0; ks < KQ / 32; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bp[ks * 4], ap[ks * 4], acc, 0, 0, 0);
#pragma unroll
  for (int r = 0; r < 4; ++r) part[w][r][lane] = acc[r];
  __syncthreads();
  if (w == 0) {
    // C layout: lane holds token (column) c16, features 4 gq + r
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float v = ((part[0][r][lane] + part[1][r][lane]) + part[2][r][lane]) + part[3][r][lane];
      const int f = f0 + 4 * gq + r;
      if (c16 < N && f < Nout) {
        const float vr = bf16_to_f32(f32_to_bf16(v));
        C[(int64_t)c16 * Nout + f] = f32_to_bf16(apply_act(act, vr));
      }
    }
  }
}

bool linear_skinny_supported(int64_t N, int K, int dtype) { return dtype == D2DMOE_BF16 && N >= 1 && N <= 16 && K % 128 == 0; }

hipError_t launch_linear_skinny(const void* A, const void* B, void* C, int N, int K, int Nout, int act, hipStream_t s) {
  hipLaunchKernelGGL(linear_skinny_kernel, dim3((Nout + 15) / 16), dim3(256), 0, s, (const bf16_t*)A, (const bf16_t*)B,
                     (bf16_t*)C, N, K, Nout, act);
  return hipGetLastError();
}

}  // namespace d2dmoe
