// Experts on MFMA as two tiled products with the hidden activations kept in memory between them.  Serves gated experts
// (Gemma shape) at more than 16 tokens, ungated experts whose width the fused sweep is not built for, and every
// float32 layer (bf16 storage: v_mfma_f32_32x32x16_bf16; float32 storage: v_mfma_f32_32x32x2_f32, float32 throughout):
//
//   up    gated:   H^T[hidden, token] = act(Wg^T . X^T) * (Wu^T . X^T) * routing[token, expert(hidden)]
//                  (ExecuteAllExperts with intermediate gating, moe_layers.py:71-78, 91-96)
//         ungated: H^T[hidden, token] = act(W1^T . X^T + b1) * routing[token, expert(hidden)]
//                  (CustomKernelExperts.forward_all, moe_layers.py:116-133)
//         -- in both cases restricted to the routed pairs by the routing factor
//   down  OUT[token, :] = sum over hidden of H[token, hidden] . W2[hidden, :]  (+ last_bias, + x)
//
// With D = 2048 neither a token tile's x rows nor its output accumulators fit next to each other on a CU, and the
// expert weights (201 MB) dwarf the activations, so the fused token-stationary sweep of the ViT shape does not carry
// over; under the dynk_max rule most experts are active for most tokens, so computing whole tiles and multiplying by
// the routing value wastes little.  The sum over hidden units runs in ascending order inside one float32 accumulator
// (per K split), which is the ascending-expert order of the reference's merge kernel (moe_impls.py:485-514).
//
// One kernel template serves both products.  Workgroup = 4 waves (2 x 2), tile = 256 tokens x 256 rows/columns of the
// weight operand, wave tile 128 x 128 = 16 accumulator tiles of 32 x 32 (256 AGPRs).  The token operand (x, or H) goes
// through LDS in fragment order, double-buffered, four fragments of K per stage; the weight operand is read straight
// from its packed fragment stream through a register ring refilled one stage ahead.  One LDS-only barrier per stage.
//
// A fragment is 64 lanes x 16 bytes: lane (c = lane % 32, g = lane / 32) holds row/column c and, in bf16, the 8 K values
// 8g .. 8g+7 of a 16-wide K step (one MFMA); in float32 the 4 K values 4g .. 4g+3 of an 8-wide K group, consumed by four
// MFMAs of K = 2 that pair value i of the g = 0 lanes with value i of the g = 1 lanes (any pairing is a valid order of
// the K sum as long as both operands use it).  Byte for byte the two element types share every layout below.
//
// The up product is computed transposed so that each lane ends up with ONE token and 16 hidden units per tile, which
// already is the A-fragment arrangement of the down product: in bf16 accumulator rows r = 8k .. 8k+7 form one fragment
// (k order: slot (g, i) <-> hidden 16*kstep + 8*(i/4) + 4g + i%4, baked into the packed W2 fragments); in float32 rows
// r = 4q .. 4q+3 form the fragment of K group q in natural order.  H is therefore written as 1 KB fragments, fully
// coalesced, and staged into LDS by the down product with straight copies.
#include "mfma_common.hpp"

namespace d2dmoe {

constexpr int GM_BT = 256;         // tokens per workgroup tile
constexpr int GM_SLAB = 8192;      // tokens per pass: bounds the workspace (H fragments + float32 partial sums)
constexpr int GM_MAX_SPLIT = 8;

typedef float f32x4v __attribute__((ext_vector_type(4)));

// Per element type: K values per fragment, elements per 16-byte piece.
template <typename T> struct GemmElem;
template <> struct GemmElem<bf16_t> { static constexpr int KPF = 16, EPP = 8; };
template <> struct GemmElem<float> { static constexpr int KPF = 8, EPP = 4; };
template <> struct GemmElem<f16_t> { static constexpr int KPF = 16, EPP = 8; };   // v_mfma_f32_32x32x16_f16: bf16's shapes

static inline int gemm_kpf(const d2dmoe_shape& sh) { return sh.dtype == D2DMOE_F32 ? 8 : 16; }
static inline size_t gemm_esize(const d2dmoe_shape& sh) { return sh.dtype == D2DMOE_F32 ? 4 : 2; }

struct GemmLayout {
  int edp;   // neurons per expert in the hidden index space: Ed itself when it is a multiple of 4 (every group of 4
             // accumulator rows then belongs to one expert), else Ed padded to a multiple of 32
  int hp;    // padded hidden size: a multiple of 128 (gated) or 256 (ungated), the hidden units one workgroup covers
  size_t up_off, dn_off, b_off, total;
};

static GemmLayout gemm_layout(const d2dmoe_shape& sh) {
  GemmLayout L;
  const size_t es = gemm_esize(sh);
  L.edp = (sh.expert_dim % 4 == 0) ? sh.expert_dim : (sh.expert_dim + 31) / 32 * 32;
  const int quantum = sh.gated ? 128 : 256;
  L.hp = (sh.n_experts * L.edp + quantum - 1) / quantum * quantum;
  L.up_off = 0;
  L.dn_off = (size_t)L.hp * (sh.gated ? 2 : 1) * sh.d_model * es;
  L.b_off = L.dn_off + (size_t)L.hp * sh.d_model * es;
  L.total = (L.b_off + (size_t)L.hp * es + 255) / 256 * 256;
  return L;
}

bool mfma_gemm_supported(const d2dmoe_shape& sh) {
  return (sh.dtype == D2DMOE_BF16 || sh.dtype == D2DMOE_F32 || sh.dtype == D2DMOE_F16) && sh.d_model % 256 == 0 &&
         sh.d_model >= 256;
}

size_t mfma_gemm_packed_bytes(const d2dmoe_shape& sh) { return mfma_gemm_supported(sh) ? gemm_layout(sh).total : 0; }

struct GemmPlan {
  int slab;      // tokens per pass
  int n_ttiles;  // 256-token tiles per (full) pass
  int ksplit;    // K splits of the down product
  size_t h_bytes, partial_bytes;
};

static GemmPlan gemm_plan(const d2dmoe_shape& sh) {
  const GemmLayout L = gemm_layout(sh);
  GemmPlan P;
  P.slab = (int)(sh.n_tokens < GM_SLAB ? sh.n_tokens : GM_SLAB);
  P.n_ttiles = (P.slab + GM_BT - 1) / GM_BT;
  // the down product has n_ttiles * D/256 tiles; split K until the machine is covered (the fragments of every split
  // must still be whole stages of 4)
  const int tiles = P.n_ttiles * (sh.d_model / 256);
  const int ks2 = L.hp / gemm_kpf(sh);
  P.ksplit = 1;
  while (P.ksplit < GM_MAX_SPLIT && tiles * P.ksplit < device_cu_count() && (ks2 / (P.ksplit * 2)) % 4 == 0) P.ksplit *= 2;
  P.h_bytes = ((size_t)P.n_ttiles * GM_BT * L.hp * gemm_esize(sh) + 255) / 256 * 256;
  P.partial_bytes = ((size_t)P.ksplit * P.slab * sh.d_model * 4 + 255) / 256 * 256;
  return P;
}

size_t mfma_gemm_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_gemm_supported(sh) || sh.n_tokens <= 0) return 0;
  const GemmPlan P = gemm_plan(sh);
  return P.h_bytes + P.partial_bytes;
}

// ---------------------------------------------------------------------------------------------------
// Packing (lane = 32 g + c).  KPF = K values per fragment (16 bf16 / 8 float32), EPP = elements per lane (8 / 4),
// KS = D/KPF, KS2 = HP/KPF; hidden index h = e*EdP + j, zero beyond Ed and beyond E.
//   up stream   gated:   [hidden block HP/64][fragment KS][tile 4: gate 0,1, up 0,1][lane][EPP]   A fragment:
//                        row h = 64*block + 32*(tile%2) + c,  d = KPF*fragment + EPP*g + i          value w[e][d][j]
//               ungated: [hidden block HP/128][fragment KS][tile 4][lane][EPP]:  row h = 128*block + 32*tile + c
//   down stream [column block D/128][fragment KS2][tile 4][lane][EPP]                   B fragment:
//               column = 128*block + 32*tile + c;  bf16: h = 16*fragment + 8*(i/4) + 4g + i%4,
//               float32: h = 8*fragment + 4g + i                                         value w2[e][j][column]
//   bias        [HP] (ungated; zeros when the experts have none)
// ---------------------------------------------------------------------------------------------------
template <typename T>
__global__ void pack_gemm_kernel(const T* __restrict__ wg, const T* __restrict__ wu, const T* __restrict__ wd,
                                 const T* __restrict__ b1, T* __restrict__ dup, T* __restrict__ ddn, T* __restrict__ db, int D,
                                 int E, int Ed, int edp, int hp, int gated) {
  constexpr int KPF = GemmElem<T>::KPF, EPP = GemmElem<T>::EPP;
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int KS = D / KPF, KS2 = hp / KPF;
  const int hb = gated ? 64 : 128;   // hidden units per block of the up stream
  const int64_t n_up = (int64_t)(hp / hb) * KS * 4 * 64;
  const int64_t n_dn = (int64_t)(D / 128) * KS2 * 4 * 64;
  if (p < n_up) {
    int64_t q = p;
    const int lane = (int)(q % 64); q /= 64;
    const int tile = (int)(q % 4); q /= 4;
    const int ks = (int)(q % KS);
    const int blk = (int)(q / KS);
    const int g = lane >> 5, c = lane & 31;
    const int h = gated ? (64 * blk + 32 * (tile & 1) + c) : (128 * blk + 32 * tile + c);
    const int e = h / edp, j = h % edp;
    const T* src = (gated && tile >= 2) ? wu : wg;
    const bool ok = e < E && j < Ed;
#pragma unroll
    for (int i = 0; i < EPP; ++i) {
      const int d = KPF * ks + EPP * g + i;
      dup[p * EPP + i] = ok ? src[((int64_t)e * D + d) * Ed + j] : (T)0;
    }
  } else if (p < n_up + n_dn) {
    const int64_t pp = p - n_up;
    int64_t q = pp;
    const int lane = (int)(q % 64); q /= 64;
    const int tile = (int)(q % 4); q /= 4;
    const int ks2 = (int)(q % KS2);
    const int blk = (int)(q / KS2);
    const int g = lane >> 5, c = lane & 31;
    const int col = 128 * blk + 32 * tile + c;
#pragma unroll
    for (int i = 0; i < EPP; ++i) {
      const int h = (EPP == 8) ? (16 * ks2 + 8 * (i / 4) + 4 * g + (i % 4)) : (8 * ks2 + 4 * g + i);
      const int e = h / edp, j = h % edp;
      ddn[pp * EPP + i] = (e < E && j < Ed) ? wd[((int64_t)e * Ed + j) * D + col] : (T)0;
    }
  } else if (p < n_up + n_dn + hp) {
    const int h = (int)(p - n_up - n_dn);
    const int e = h / edp, j = h % edp;
    db[h] = (b1 != nullptr && e < E && j < Ed) ? b1[(int64_t)e * Ed + j] : (T)0;
  }
}

template <typename T>
static hipError_t launch_gemm_pack_t(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                                     void* packed_section, hipStream_t s) {
  constexpr int KPF = GemmElem<T>::KPF;
  const GemmLayout L = gemm_layout(sh);
  char* base = (char*)packed_section;
  const int hb = sh.gated ? 64 : 128;
  const int64_t n = (int64_t)(L.hp / hb) * (sh.d_model / KPF) * 256 + (int64_t)(sh.d_model / 128) * (L.hp / KPF) * 256 + L.hp;
  hipLaunchKernelGGL(pack_gemm_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const T*)w1, (const T*)w_up,
                     (const T*)w2, (const T*)b1, (T*)(base + L.up_off), (T*)(base + L.dn_off), (T*)(base + L.b_off), sh.d_model,
                     sh.n_experts, sh.expert_dim, L.edp, L.hp, sh.gated);
  return hipGetLastError();
}

hipError_t launch_gemm_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            void* packed_section, hipStream_t s) {
  if (sh.dtype == D2DMOE_F32) return launch_gemm_pack_t<float>(sh, w1, b1, w2, w_up, packed_section, s);
  if (sh.dtype == D2DMOE_F16) return launch_gemm_pack_t<f16_t>(sh, w1, b1, w2, w_up, packed_section, s);
  return launch_gemm_pack_t<bf16_t>(sh, w1, b1, w2, w_up, packed_section, s);
}

// ---------------------------------------------------------------------------------------------------
template <typename T>
struct GemmArgs {
  const T* x;              // [N, D] rows of this pass
  const T* routing;        // [N, E]
  const u32x4* w;          // packed weight stream of this product (fragments of 16 bytes per lane)
  const T* bias;           // [HP] first-layer bias (ungated)
  u32x4* hfrag;            // [token tile N/32][fragment HP/KPF][lane] hidden activations as A fragments
  float* partial;          // [ksplit][N][D] float32 sums of the down product
  int N; int D; int E; int edp; int hp; int act;
  int n_ttiles;            // 256-token tiles
  int tpx;                 // token tiles per XCD: ceil(n_ttiles / 8)
  int ksplit;
  const int* skip_flag;    // optional device flag: non-zero = another path has handled this call
};

// one fragment pair into a 32 x 32 accumulator tile
template <typename T>
__device__ __forceinline__ void frag_mfma(const u32x4& a, const u32x4& b, f32x16& c) {
  if constexpr (sizeof(T) == 2 && Elem<T>::dtype == D2DMOE_F16) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    f16x8 av, bv;
    __builtin_memcpy(&av, &a, 16);
    __builtin_memcpy(&bv, &b, 16);
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, c, 0, 0, 0);
  } else if constexpr (sizeof(T) == 2) {
    bf16x8 av, bv;
    __builtin_memcpy(&av, &a, 16);
    __builtin_memcpy(&bv, &b, 16);
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, c, 0, 0, 0);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[i]), __uint_as_float(b[i]), c, 0, 0, 0);
  }
}

// MODE 0: up product (weights = A operand, x = B operand through LDS); MODE 1: down product (H = A operand through
// LDS, weights = B operand).
template <typename T, int MODE, int ACT, bool GATED>
__global__ __launch_bounds__(256, 1) void gated_gemm_kernel(const GemmArgs<T> A) {
  constexpr int KPF = GemmElem<T>::KPF, EPP = GemmElem<T>::EPP;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  if (A.skip_flag != nullptr && *A.skip_flag != 0) return;   // uniform over the whole grid
  u32x4* lds0 = (u32x4*)smem_raw;            // [8 token tiles][4 fragments][64 lanes]
  u32x4* lds1 = lds0 + 8 * 4 * 64;
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int wm = w >> 1, wn = w & 1;         // half of the weight rows/columns, half of the tokens
  const int g = lane >> 5, c32 = lane & 31;
  // Workgroups are dealt to the 8 XCDs round-robin.  An XCD keeps "its" token tiles (tpx of them) and walks the weight
  // blocks, so at any time its L2 holds a few token tiles and one set of weight blocks shared by all of its CUs.
  const int xcd = blockIdx.x & 7, kk = blockIdx.x >> 3;
  const int tt = xcd + 8 * (kk % A.tpx);
  int nb = kk / A.tpx;
  if (tt >= A.n_ttiles) return;
  int split = 0;
  if (MODE == 1) { split = nb % A.ksplit; nb /= A.ksplit; }
  const int N = A.N, D = A.D;
  const int KS2T = A.hp / KPF;                                    // fragments along K of the whole down product
  const int n_ks = (MODE == 0) ? (D / KPF) : (KS2T / A.ksplit);   // ... of this workgroup
  const int ks_begin = (MODE == 0) ? 0 : split * n_ks;
  const int S = n_ks / 4;                                         // stages
  const int KST = (MODE == 0) ? (D / KPF) : KS2T;
  const u32x4* wbase = A.w + ((int64_t)(nb * 2 + wm) * KST + ks_begin) * 256 + lane;

  f32x16 acc[4][4];   // [weight tile][token tile]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- token operand: global -> registers -> LDS, 8 pieces of 16 bytes per thread and stage
  u32x4 xv[8];
  const int xrow = t >> 3, xpc = t & 7;   // MODE 0: row within a 32-token tile, 16-byte piece of the stage's K slice
  // MODE 0 stores 8 pieces of one row per 8 lanes; inside a fragment the row slot is XORed with the piece index (and
  // bit 3 with the row's parity) so that those stores spread over all LDS banks.  A read of fragment (index, half)
  // applies the same XOR, which only permutes its 32 consecutive slots.
  int xoff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
    xoff[ks] = (MODE == 0) ? (32 * g + (c32 ^ (2 * ks + g) ^ ((c32 & 1) << 3))) : lane;
  auto load_x = [&](int s) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (MODE == 0) {
        int64_t tok = (int64_t)tt * GM_BT + i * 32 + xrow;
        tok = tok < N ? tok : (N - 1);   // rows beyond N repeat the last row; their H is forced to zero below
        xv[i] = *(const u32x4*)(A.x + tok * D + s * (4 * KPF) + xpc * EPP);
      } else {
        xv[i] = A.hfrag[(((int64_t)tt * 8 + i) * KS2T + ks_begin + s * 4 + w) * 64 + lane];
      }
    }
  };
  auto store_x = [&](u32x4* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (MODE == 0) buf[(i * 4 + (xpc >> 1)) * 64 + 32 * (xpc & 1) + (xrow ^ xpc ^ ((xrow & 1) << 3))] = xv[i];
      else buf[i * 256 + t] = xv[i];
    }
  };
  // ---- weight operand: a register ring of 16 fragments (one stage); a slot is refilled with the fragment one stage
  // ahead as soon as it has been handed to the MFMAs
  u32x4 ring[4][4];   // [fragment][tile]
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
#pragma unroll
    for (int i = 0; i < 4; ++i) ring[ks][i] = wbase[(ks * 4 + i) * 64];
  auto compute = [&](const u32x4* buf, int s_next) __attribute__((always_inline)) {
    const u32x4* xl = buf + (wn * 4) * 4 * 64;
    const u32x4* wn_ = wbase + (int64_t)s_next * 16 * 64;
    u32x4 xb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xb[j] = xl[(j * 4 + 0) * 64 + xoff[0]];
    static_for<0, 4>([&](auto ks_c) __attribute__((always_inline)) {
      constexpr int ks = decltype(ks_c)::value;
      constexpr int kn = (ks + 1 < 4) ? ks + 1 : ks;
      u32x4 wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        wv[i] = ring[ks][i];
        ring[ks][i] = wn_[(ks * 4 + i) * 64];
      }
      u32x4 nxb[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) nxb[j] = xl[(j * 4 + kn) * 64 + xoff[kn]];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (MODE == 0) frag_mfma<T>(wv[i], xb[j], acc[i][j]);
          else frag_mfma<T>(xb[j], wv[i], acc[i][j]);
        }
#pragma unroll
      for (int j = 0; j < 4; ++j) xb[j] = nxb[j];
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  load_x(0);
  store_x(lds0);
  __syncthreads();
  for (int s = 0; s < S; ++s) {
    u32x4* cur = (s & 1) ? lds1 : lds0;
    u32x4* nxt = (s & 1) ? lds0 : lds1;
    const bool more = s + 1 < S;
    if (more) load_x(s + 1);
    __builtin_amdgcn_sched_barrier(0);
    compute(cur, more ? s + 1 : s);   // the last stage re-reads its own fragments: in bounds, unused
    if (more) store_x(nxt);
    lds_barrier();
  }

  if (MODE == 0) {
    // gated: weight tiles 0,1 = gate rows, 2,3 = up rows of the same 64 hidden units; ungated: four tiles of 32 hidden
    // units.  lane = token c32 of token tile j; accumulator row r = hidden unit 8*(r/4) + 4g + r%4 of the tile
    constexpr int NH = GATED ? 2 : 4;          // hidden tiles per wave
    constexpr int HW = GATED ? 64 : 128;       // hidden units per wave
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tl = wn * 4 + j;
      const int64_t tok = (int64_t)tt * GM_BT + tl * 32 + c32;
#pragma unroll
      for (int i = 0; i < NH; ++i) {
        const int h0 = (nb * 2 + wm) * HW + 32 * i;
        // experts of a multiple of 32 neurons: the whole 32-row tile belongs to one expert, one routing value serves it
        const bool one_expert = (A.edp & 31) == 0;   // uniform
        float rw_tile = 0.f;
        bool live_tile = false;
        if (one_expert) {
          const int e = h0 / A.edp;
          live_tile = tok < N && e < A.E;
          rw_tile = live_tile ? Elem<T>::load(A.routing + tok * A.E + e) : 0.f;
        }
        float hv[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float rw = rw_tile;
          bool live = live_tile;
          if (!one_expert) {
            const int e = (h0 + 8 * q + 4 * g) / A.edp;   // the expert of these four rows
            live = tok < N && e < A.E;
            rw = live ? Elem<T>::load(A.routing + tok * A.E + e) : 0.f;
          }
          float bq[4] = {0.f, 0.f, 0.f, 0.f};
          if (!GATED) {
#pragma unroll
            for (int u = 0; u < 4; ++u) bq[u] = Elem<T>::load(A.bias + h0 + 8 * q + 4 * g + u);
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int r = 4 * q + u;
            const float pre = GATED ? acc[i][j][r] : (acc[i][j][r] + bq[u]);
            const float gv = (ACT >= 0) ? act_fn<ACT>(pre) : apply_act(A.act, pre);
            const float v = (GATED ? gv * acc[2 + (i & 1)][j][r] : gv) * rw;
            hv[r] = (live && rw != 0.f) ? v : 0.f;
          }
        }
        u32x4* hdst = A.hfrag + (((int64_t)tt * 8 + tl) * KS2T + h0 / KPF) * 64 + lane;
        if constexpr (sizeof(T) == 2) {
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            u32x4 pk;
            pk.x = pack2_16<T>(hv[8 * k + 0], hv[8 * k + 1]); pk.y = pack2_16<T>(hv[8 * k + 2], hv[8 * k + 3]);
            pk.z = pack2_16<T>(hv[8 * k + 4], hv[8 * k + 5]); pk.w = pack2_16<T>(hv[8 * k + 6], hv[8 * k + 7]);
            hdst[k * 64] = pk;
          }
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            u32x4 pk;
            pk.x = __float_as_uint(hv[4 * q + 0]); pk.y = __float_as_uint(hv[4 * q + 1]);
            pk.z = __float_as_uint(hv[4 * q + 2]); pk.w = __float_as_uint(hv[4 * q + 3]);
            hdst[q * 64] = pk;
          }
        }
      }
    }
  } else {
    // lane = column c32 of weight tile i; accumulator row r = token 8*(r/4) + 4g + r%4 of token tile j
    float* pbase = A.partial + (int64_t)split * N * D;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = (nb * 2 + wm) * 128 + 32 * i + c32;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t tok0 = (int64_t)tt * GM_BT + (wn * 4 + j) * 32 + 4 * g;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t tok = tok0 + 8 * (r / 4) + (r % 4);
          if (tok < N) pbase[tok * D + col] = acc[i][j][r];
        }
      }
    }
  }
}

// out[n, :] = round(sum over splits (ascending) + last_bias + x), 8 columns per thread
template <typename T>
__global__ __launch_bounds__(256) void gemm_finish_kernel(const float* __restrict__ partial, const T* __restrict__ last_bias,
                                                          const T* __restrict__ x, T* __restrict__ out, int64_t N, int D,
                                                          int ksplit, int add_residual, const int* __restrict__ skip_flag) {
  if (skip_flag != nullptr && *skip_flag != 0) return;   // uniform over the whole grid
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_row = D / 8;
  if (p >= N * per_row) return;
  const int64_t n = p / per_row;
  const int col = (int)(p % per_row) * 8;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = 0.f;
  for (int s = 0; s < ksplit; ++s) {
    const float4 a = *(const float4*)(partial + ((int64_t)s * N + n) * D + col);
    const float4 b = *(const float4*)(partial + ((int64_t)s * N + n) * D + col + 4);
    v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
  }
  if (last_bias != nullptr) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += Elem<T>::load(last_bias + col + i);
  }
  if (add_residual) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += Elem<T>::load(x + n * D + col + i);
  }
  if constexpr (sizeof(T) == 2) {
    uint4 o;
    o.x = pack2_16<T>(v[0], v[1]); o.y = pack2_16<T>(v[2], v[3]);
    o.z = pack2_16<T>(v[4], v[5]); o.w = pack2_16<T>(v[6], v[7]);
    *(uint4*)(out + n * D + col) = o;
  } else {
    *(float4*)(out + n * D + col) = float4{v[0], v[1], v[2], v[3]};
    *(float4*)(out + n * D + col + 4) = float4{v[4], v[5], v[6], v[7]};
  }
}

template <typename T>
static hipError_t launch_sum_partials_t(const float* partial, const void* last_bias, const void* x, void* out, int64_t N, int D,
                                        int n_splits, int add_residual, hipStream_t s, const int* skip_flag = nullptr) {
  const int64_t items = N * (D / 8);
  hipLaunchKernelGGL(gemm_finish_kernel<T>, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s, partial, (const T*)last_bias,
                     (const T*)x, (T*)out, N, D, n_splits, add_residual, skip_flag);
  return hipGetLastError();
}

hipError_t launch_sum_partials(const float* partial, const void* last_bias, const void* x, void* out, int64_t N, int D,
                               int n_splits, int add_residual, hipStream_t s, int dtype, const int* skip_flag) {
  if (dtype == D2DMOE_F16)
    return launch_sum_partials_t<f16_t>(partial, last_bias, x, out, N, D, n_splits, add_residual, s, skip_flag);
  return launch_sum_partials_t<bf16_t>(partial, last_bias, x, out, N, D, n_splits, add_residual, s, skip_flag);
}

template <typename T, int ACT, bool GATED>
static hipError_t launch_gemm_act(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                                  const void* last_bias, void* out, void* workspace, hipStream_t s, const int* skip_flag) {
  const GemmLayout L = gemm_layout(sh);
  const GemmPlan P = gemm_plan(sh);
  const char* pk = (const char*)packed_section;
  const size_t lds = 2 * 8 * 4 * 64 * 16;
  auto k_up = gated_gemm_kernel<T, 0, ACT, GATED>;
  auto k_dn = gated_gemm_kernel<T, 1, -1, true>;
  hipError_t e = hipFuncSetAttribute((const void*)k_up, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  e = hipFuncSetAttribute((const void*)k_dn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  for (int64_t t0 = 0; t0 < sh.n_tokens; t0 += P.slab) {
    const int n = (int)((sh.n_tokens - t0) < P.slab ? (sh.n_tokens - t0) : P.slab);
    GemmArgs<T> A;
    A.x = (const T*)x + t0 * sh.d_model;
    A.routing = (const T*)routing + t0 * sh.n_experts;
    A.bias = (const T*)(pk + L.b_off);
    A.hfrag = (u32x4*)workspace;
    A.partial = (float*)((char*)workspace + P.h_bytes);
    A.N = n; A.D = sh.d_model; A.E = sh.n_experts; A.edp = L.edp; A.hp = L.hp; A.act = sh.activation;
    A.n_ttiles = (n + GM_BT - 1) / GM_BT;
    A.tpx = (A.n_ttiles + 7) / 8;
    A.ksplit = P.ksplit;
    A.skip_flag = skip_flag;
    A.w = (const u32x4*)(pk + L.up_off);
    hipLaunchKernelGGL(k_up, dim3((unsigned)(8 * A.tpx * (L.hp / (GATED ? 128 : 256)))), dim3(256), lds, s, A);
    A.w = (const u32x4*)(pk + L.dn_off);
    hipLaunchKernelGGL(k_dn, dim3((unsigned)(8 * A.tpx * (sh.d_model / 256) * P.ksplit)), dim3(256), lds, s, A);
    e = launch_sum_partials_t<T>(A.partial, last_bias, A.x, (T*)out + t0 * sh.d_model, (int64_t)n, sh.d_model, P.ksplit,
                                 sh.add_residual, s, skip_flag);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <typename T, bool GATED>
static hipError_t launch_gemm_gated(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                                    const void* last_bias, void* out, void* workspace, hipStream_t s, const int* skip_flag) {
  switch (sh.activation) {
    case D2DMOE_ACT_RELU: return launch_gemm_act<T, D2DMOE_ACT_RELU, GATED>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
    case D2DMOE_ACT_GELU: return launch_gemm_act<T, D2DMOE_ACT_GELU, GATED>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
    case D2DMOE_ACT_GELU_TANH: return launch_gemm_act<T, D2DMOE_ACT_GELU_TANH, GATED>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
    case D2DMOE_ACT_SILU: return launch_gemm_act<T, D2DMOE_ACT_SILU, GATED>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
    default: return launch_gemm_act<T, -1, GATED>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
  }
}

hipError_t launch_mfma_gemm(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                            const void* last_bias, void* out, void* workspace, hipStream_t s, const int* skip_flag) {
  if (sh.dtype == D2DMOE_F32) {
    if (sh.gated) return launch_gemm_gated<float, true>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
    return launch_gemm_gated<float, false>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
  }
  if (sh.dtype == D2DMOE_F16) {
    if (sh.gated) return launch_gemm_gated<f16_t, true>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
    return launch_gemm_gated<f16_t, false>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
  }
  if (sh.gated) return launch_gemm_gated<bf16_t, true>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
  return launch_gemm_gated<bf16_t, false>(sh, x, routing, packed_section, last_bias, out, workspace, s, skip_flag);
}

}  // namespace d2dmoe
