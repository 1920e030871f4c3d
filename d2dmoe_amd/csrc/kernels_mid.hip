// Compacted bf16 MFMA path for routing of low to middling density (one to a few dozen experts per token), where a token
// tile touches every expert but each expert only a fraction of the tile's tokens.  Work follows the routed
// (token, expert) pairs, as in the reference's grouped kernels (moe_impls.py:124-133, 270-293), and no output row is
// written per pair:
//
//   plan      per segment of 32 tokens the routed-token count per expert and its prefix over segments (shared with the
//             expert-major path); per tile of 256 tokens the number of 16-pair groups; then a scatter that lists every
//             pair twice over: in the expert-major order (expert ascending, tokens ascending inside an expert) its token
//             and the row its hidden values go to, the rows being laid out tile-major (tile, expert, token), every
//             (tile, expert) run padded to a multiple of 16 rows
//   up        expert-stationary first layer.  Two waves share an expert's W1 fragments (each one half of K, 96 registers)
//             and walk a range of the expert-major list in groups of 16 pairs; the 16 x rows of a group are the B operand
//             of v_mfma_f32_16x16x32_bf16, fetched straight into registers one group ahead.  The two halves' sums meet in
//             LDS; bias, activation, routing weight, rounding; 32 bf16 per pair go to the pair's row (element 31 carries the
//             token's row inside its tile instead: experts hold at most 31 neurons here)
//   down      output-stationary second layer.  A workgroup owns 256 tokens x 128 output columns as float32 in LDS and walks
//             the tile's rows in memory order (expert ascending): per 16 rows one MFMA per wave against the expert's W2^T
//             fragment, whose 16 x 16 result is added to the rows of its tokens.  A wave owns its columns exclusively, so
//             every output element is summed by one wave in program order: ascending expert order in float32, one rounding
//             after + last_bias (+ x) -- deterministic, the order of the reference's merge kernel (moe_impls.py:499-514).
//
// Fragment layouts of the 16x16x32 bf16 MFMA on a 64-lane wave (q = lane / 16, c = lane % 16):
//   A (16 x 32): lane holds row c,    k = 8q .. 8q+7         B (32 x 16): lane holds column c, k = 8q .. 8q+7
//   C (16 x 16): lane holds column c, rows 4q + r, r = 0..3
#include "mfma_common.hpp"

namespace d2dmoe {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int MID_T2 = 256;                  // tokens per tile of the second layer
constexpr int MID_T2_SEGS = MID_T2 / SP_SEG; // plan segments per tile
constexpr int MID_DS = 128;                  // output columns per workgroup of the second layer
constexpr int MID_OS = MID_DS + 4;           // row stride of the float32 output tile (rows shift by 4 banks)
constexpr int MID_RING = 32;                 // 1 KB units of the second layer kept in flight per wave
constexpr int MID_UP_THREADS = 512;
constexpr int MID_DOWN_THREADS = 512;
static_assert(MID_T2 % SP_SEG == 0 && MID_T2 <= 256, "a token's row inside its tile fits 8 bits");

bool mfma_mid_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 || sh.gated) return false;
  if (sh.d_model != 768) return false;
  // element 31 of a hidden row carries the token's row inside its tile; the plan keeps one lane per expert, 4 per wave
  return sh.expert_dim < MID_HROW && sh.n_experts <= 256;
}

struct MidWorkspace {
  int64_t n_seg, n_tiles, cap, cap_rows;
  size_t seg_counts, seg_offsets, totals, seg_pairs, offsets, flag, tile_groups, rec, hc, total;
};

static MidWorkspace mid_workspace(const d2dmoe_shape& sh) {
  MidWorkspace W;
  const int64_t N = sh.n_tokens;
  const int E = sh.n_experts;
  W.n_seg = cdiv64(N, SP_SEG);
  W.n_tiles = cdiv64(N, MID_T2);
  W.cap = N * (int64_t)(E < MID_MAX_MEAN_K ? E : MID_MAX_MEAN_K);
  W.cap_rows = W.cap + 16 * W.n_tiles * E;   // every (tile, expert) run ends on a multiple of 16 rows
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += (bytes + 255) / 256 * 256; return o; };
  W.seg_counts = take((size_t)W.n_seg * E * 4);
  W.seg_offsets = take((size_t)W.n_seg * E * 4);
  W.totals = take((size_t)E * 4);
  W.seg_pairs = take((size_t)W.n_seg * 4);
  W.offsets = take((size_t)(E + 1) * 4);
  W.flag = take(16);
  W.tile_groups = take((size_t)W.n_tiles * 4);
  W.rec = take((size_t)W.cap * 8);
  W.hc = take((size_t)W.cap_rows * MID_HROW * 2);
  W.total = off;
  return W;
}

size_t mfma_mid_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_mid_supported(sh) || sh.n_tokens <= 0) return 0;
  return mid_workspace(sh).total;
}

int64_t mfma_mid_capacity_pairs(const d2dmoe_shape& sh) { return mid_workspace(sh).cap; }

// ---------------------------------------------------------------------------------------------------
// Packing.  Experts are padded to 32 neurons with zero weights (and zero bias, in the expert-major section's bias table).
//   W1 fragments   [E][kstep D/32][row tile 2][lane][8]:  neuron j = rt*16 + c, d = kstep*32 + 8q + i     w1[e][d][j]
//   W2^T fragments [E][column tile D/16][lane][8]:        column = ct*16 + c,   neuron k = 8q + i         w2[e][k][column]
// ---------------------------------------------------------------------------------------------------
__global__ void pack_mid_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ w2, bf16_t* __restrict__ d1,
                                bf16_t* __restrict__ d2, int D, int E, int Ed) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int KS = D / 32, CT = D / 16;
  const int64_t n1 = (int64_t)E * KS * 2 * 64, n2 = (int64_t)E * CT * 64;
  const int lane = (int)(p % 64);
  const int q = lane / 16, c = lane % 16;
  if (p < n1) {
    int64_t r = p / 64;
    const int rt = (int)(r % 2); r /= 2;
    const int ks = (int)(r % KS);
    const int e = (int)(r / KS);
    const int j = rt * 16 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 32 + 8 * q + i;
      d1[p * 8 + i] = (j < Ed) ? w1[((int64_t)e * D + d) * Ed + j] : (bf16_t)0;
    }
  } else if (p < n1 + n2) {
    const int64_t pp = p - n1;
    const int64_t r = pp / 64;
    const int ct = (int)(r % CT);
    const int e = (int)(r / CT);
    const int col = ct * 16 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = 8 * q + i;
      d2[pp * 8 + i] = (k < Ed) ? w2[((int64_t)e * Ed + k) * D + col] : (bf16_t)0;
    }
  }
}

hipError_t launch_mid_pack(const d2dmoe_shape& sh, const PackedLayout& L, const void* w1, const void* w2, void* packed,
                           hipStream_t s) {
  char* base = (char*)packed;
  const int64_t n = (int64_t)sh.n_experts * (sh.d_model / 32) * 2 * 64 + (int64_t)sh.n_experts * (sh.d_model / 16) * 64;
  hipLaunchKernelGGL(pack_mid_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)w1, (const bf16_t*)w2,
                     (bf16_t*)(base + L.m1_off), (bf16_t*)(base + L.m2_off), sh.d_model, sh.n_experts, sh.expert_dim);
  return hipGetLastError();
}

struct MidArgs {
  const bf16_t* x; const bf16_t* routing; const bf16x8* w1f; const bf16x8* w2f; const bf16_t* b1s;
  const int32_t* seg_offsets; const int32_t* totals; int32_t* offsets; int32_t* flag; int32_t* tile_groups; int2* rec;
  bf16_t* hc; const bf16_t* last_bias; bf16_t* out;
  int64_t N; int64_t cap; int E; int n_seg; int n_tiles; int act_rt; int add_residual;
};

// Loads whose completion is waited for by hand: the compiler's own bookkeeping gives up on rings of loads carried round
// a loop (it waits for every load in flight, which serialises the kernel on memory latency).  A register written by
// one of these is touched by nothing until a wait has named it.  Loads return in the order they were issued.
__device__ __forceinline__ void load16_async(bf16x8& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
template <int OFF>
__device__ __forceinline__ void load16_async_at(bf16x8& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(dst) : "v"(p), "n"(OFF) : "memory");
}
__device__ __forceinline__ void load8_async(int2& dst, const void* p) {
  asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void load2_async(uint32_t& dst, const void* p) {
  asm volatile("global_load_ushort %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}

__device__ inline int mid_wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int t = __shfl_up(v, off, 64);
    if (lane >= off) v += t;
  }
  return v;
}

// routed tokens of expert e in segments [0, s): the scan's rows, the per-expert totals past the last segment
__device__ __forceinline__ int mid_seg_prefix(const int32_t* seg_offsets, const int32_t* totals, int64_t s, int n_seg, int E, int e) {
  return (s < n_seg) ? seg_offsets[s * E + e] : totals[e];
}

// ---------------------------------------------------------------------------------------------------
// Plan: 16-pair groups per tile of the second layer (a wave per tile, lanes = experts).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mid_tile_kernel(const int32_t* __restrict__ seg_offsets, const int32_t* __restrict__ totals,
                                                       int32_t* __restrict__ tile_groups, int E, int n_seg, int n_tiles) {
  const int lane = threadIdx.x & 63;
  const int tile = (int)((blockIdx.x * blockDim.x + threadIdx.x) / 64);
  if (tile >= n_tiles) return;
  const int64_t s0 = (int64_t)tile * MID_T2_SEGS, s1 = s0 + MID_T2_SEGS;
  int sum = 0;
  for (int e = lane; e < E; e += 64) {
    const int c = mid_seg_prefix(seg_offsets, totals, s1, n_seg, E, e) - seg_offsets[s0 * E + e];
    sum += (c + 15) >> 4;
  }
  sum = wave_sum_i32(sum);
  if (lane == 0) tile_groups[tile] = sum;
}

// ---------------------------------------------------------------------------------------------------
// Plan: scatter.  A wave per segment of 32 tokens, lanes = experts.  For every routed pair of the segment: its place in
// the expert-major list (expert offset + routed tokens of the expert in earlier segments + rank inside the segment) gets
// the token and the pair's hidden row = 16 * (groups of earlier tiles + groups of earlier experts in this tile) + rank of
// the token among the expert's routed tokens of the tile.  The first wave publishes the experts' offsets and the flag.
// ---------------------------------------------------------------------------------------------------
template <int VPT>
__global__ __launch_bounds__(256) void mid_scatter_kernel(const bf16_t* __restrict__ routing, const int32_t* __restrict__ seg_offsets,
                                                          const int32_t* __restrict__ totals, const int32_t* __restrict__ tile_groups,
                                                          int32_t* __restrict__ offsets, int32_t* __restrict__ flag,
                                                          int2* __restrict__ rec, int64_t N, int E, int n_seg, int64_t cap) {
  const int lane = threadIdx.x & 63;
  const int64_t seg = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / 64;
  if (seg >= n_seg) return;
  const int tile = (int)(seg / MID_T2_SEGS);
  const int64_t s0 = (int64_t)tile * MID_T2_SEGS, s1 = s0 + MID_T2_SEGS;
  const int64_t t0 = seg * SP_SEG;
  const int rows = (int)((N - t0) < SP_SEG ? (N - t0) : SP_SEG);
  int tot[VPT], so_seg[VPT], so_t0[VPT], so_t1[VPT];
  unsigned onbits[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int e = lane + k * 64;
    const int ec = (e < E) ? e : (E - 1);
    tot[k] = totals[ec];
    so_seg[k] = seg_offsets[seg * E + ec];
    so_t0[k] = seg_offsets[s0 * E + ec];
    so_t1[k] = (s1 < n_seg) ? seg_offsets[(s1 < n_seg ? s1 : 0) * E + ec] : tot[k];
    bf16_t v[SP_SEG];
#pragma unroll
    for (int i = 0; i < SP_SEG; ++i) {
      const int r = (i < rows) ? i : (rows - 1);
      v[i] = routing[(t0 + r) * E + ec];
    }
    onbits[k] = 0u;
#pragma unroll
    for (int i = 0; i < SP_SEG; ++i) onbits[k] |= ((i < rows && e < E && (v[i] & 0x7fff) != 0) ? 1u : 0u) << i;
  }
  int tbase = 0;   // groups of all earlier tiles
  for (int i0 = 0; i0 < tile; i0 += 64) tbase += (i0 + lane < tile) ? tile_groups[i0 + lane] : 0;
  tbase = wave_sum_i32(tbase);
  int eoff[VPT], goff[VPT];
  int run = 0, grun = 0;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int e = lane + k * 64;
    const int c = (e < E) ? tot[k] : 0;
    const int g = (e < E) ? ((so_t1[k] - so_t0[k] + 15) >> 4) : 0;
    const int ci = mid_wave_incl_scan(c, lane), gi = mid_wave_incl_scan(g, lane);
    eoff[k] = run + ci - c;
    goff[k] = grun + gi - g;
    run += __shfl(ci, 63, 64);
    grun += __shfl(gi, 63, 64);
  }
  const bool ok = (int64_t)run <= cap;
  if (seg == 0) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int e = lane + k * 64;
      if (e < E) offsets[e] = eoff[k];
    }
    if (lane == 0) {
      offsets[E] = run;
      flag[0] = ok ? 1 : 0;
    }
  }
  if (!ok) return;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    int64_t pos = (int64_t)eoff[k] + so_seg[k];
    int row = (tbase + goff[k]) * 16 + (so_seg[k] - so_t0[k]);
    unsigned bits = onbits[k];
    while (bits != 0u) {
      const int i = __ffs(bits) - 1;
      bits &= bits - 1u;
      rec[pos] = make_int2((int)(t0 + i), row);
      ++pos;
      ++row;
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// First layer.  512 threads = 4 pairs of waves; the two waves of a pair hold one half of K each of an expert's W1
// fragments (96 registers) and share a range of the 16-pair groups of the expert-major list (all experts' groups in one
// sequence, cut into equal ranges over the pairs of the whole grid: a busy expert simply spans more ranges).  A step:
// request the 12 x fragments and the routing weight of the next group and the list entries of the group three ahead,
// wait for this group's, 24 MFMAs, hand the upper half's sums over through LDS, finish the rows in the lower half's
// wave.  The steps of a workgroup run in lock step (one barrier each); all of them do the same amount of work.
// ---------------------------------------------------------------------------------------------------
template <int D, int ACT>
__global__ __launch_bounds__(MID_UP_THREADS) void mid_up_kernel(const MidArgs A) {
  constexpr int KS = D / 32, KH = KS / 2;   // K steps of 32; per wave
  static_assert(KH == 12, "operand lists below name 12 fragments");
  __shared__ int s_goff[258];               // first group of every expert in the sequence of all groups
  __shared__ int s_off[258];                // the experts' offsets in the expert-major list
  __shared__ f32x4 xch[MID_UP_THREADS / 128][2][2][64];   // [pair][step parity][row tile][lane]
  if (A.flag[0] == 0) return;               // uniform over the grid: the dense sweep runs instead
  const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int q = lane >> 4, c = lane & 15;
  const int pr = w >> 1, h = w & 1;
  const int E = A.E;
  if (w == 0) {
    int run = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int g = (e < E) ? ((A.totals[e] + 15) >> 4) : 0;
      const int gi = mid_wave_incl_scan(g, lane);
      if (e < E) s_goff[e] = run + gi - g;
      run += __shfl(gi, 63, 64);
    }
    if (lane == 0) s_goff[E] = run;
  }
  for (int e = t; e <= E; e += MID_UP_THREADS) s_off[e] = A.offsets[e];
  __syncthreads();
  const int G = s_goff[E];
  if (G == 0) return;
  const int n_pairs = gridDim.x * (MID_UP_THREADS / 128);
  const int per = (G + n_pairs - 1) / n_pairs;
  const int gp = blockIdx.x * (MID_UP_THREADS / 128) + pr;
  const int g_lo = (gp * per < G) ? gp * per : G;
  const int g_hi = (g_lo + per < G) ? g_lo + per : G;
  const int g_last = (g_hi > g_lo) ? g_hi - 1 : G - 1;    // groups past the range: this one again, nothing stored

  // list entries of a group: (expert, valid pairs, this lane's token and hidden row)
  int e_m = 0;
  {
    const int g0 = (g_lo < g_last) ? g_lo : g_last;
    while (s_goff[e_m + 1] <= g0) ++e_m;    // experts without pairs have no groups
  }
  int2 m_rec[4];
  int m_e[4], m_valid[4];
  auto issue_meta = [&](int2& dst, int& e_out, int& valid_out, int g) __attribute__((always_inline)) {
    const int gc = (g < g_last) ? g : g_last;
    while (s_goff[e_m + 1] <= gc) ++e_m;
    const int j = gc - s_goff[e_m];
    const int left = s_off[e_m + 1] - s_off[e_m] - 16 * j;
    const int valid = left < 16 ? left : 16;
    e_out = e_m;
    valid_out = (g < g_hi) ? valid : 0;
    load8_async(dst, A.rec + ((int64_t)s_off[e_m] + 16 * j + (c < valid ? c : valid - 1)));
  };
  bf16x8 xb[2][KH];
  uint32_t rwb[2];
  auto issue_x = [&](bf16x8 (&dst)[KH], uint32_t& rw, const int2& rec, int e) __attribute__((always_inline)) {
    const unsigned char* p = (const unsigned char*)(A.x + (int64_t)rec.x * D + h * (D / 2) + 8 * q);
    static_for<0, KH>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      load16_async_at<i * 64>(dst[i], p);
    });
    load2_async(rw, A.routing + (int64_t)rec.x * E + e);
  };
  constexpr int PER_STEP = KH + 2;          // loads a step issues
  auto wait_step = [&](bf16x8 (&b)[KH], uint32_t& rw, int2& rec) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(%15)"
                 : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7]), "+v"(b[8]),
                   "+v"(b[9]), "+v"(b[10]), "+v"(b[11]), "+v"(rw), "+v"(rec.x), "+v"(rec.y)
                 : "n"(PER_STEP)
                 : "memory");
  };

  // prologue: entries of the first three groups, then the x fragments of the first
  issue_meta(m_rec[0], m_e[0], m_valid[0], g_lo);
  issue_meta(m_rec[1], m_e[1], m_valid[1], g_lo + 1);
  issue_meta(m_rec[2], m_e[2], m_valid[2], g_lo + 2);
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(m_rec[0].x), "+v"(m_rec[0].y), "+v"(m_rec[1].x), "+v"(m_rec[1].y), "+v"(m_rec[2].x), "+v"(m_rec[2].y) :: "memory");
  issue_x(xb[0], rwb[0], m_rec[0], m_e[0]);

  bf16x8 wf[KH][2];
  int2 braw[2];                             // the expert's biases for this lane's neurons, bf16 pairs
  int e_w = -1;
  for (int it0 = 0; it0 < per; it0 += 4) {
    static_for<0, 4>([&](auto ph_c) __attribute__((always_inline)) {
      constexpr int ph = decltype(ph_c)::value;
      const int it = it0 + ph;
      if (it < per) {                        // uniform over the grid
        constexpr int cur = ph & 1, nxt = cur ^ 1;
        // requests: x fragments and weight of group it + 1 (its entries arrived a step ago), entries of group it + 3
        issue_x(xb[nxt], rwb[nxt], m_rec[(ph + 1) & 3], m_e[(ph + 1) & 3]);
        issue_meta(m_rec[(ph + 3) & 3], m_e[(ph + 3) & 3], m_valid[(ph + 3) & 3], g_lo + it + 3);
        wait_step(xb[cur], rwb[cur], m_rec[(ph + 2) & 3]);
        const int e = m_e[ph];
        if (e != e_w) {                      // uniform over the pair: the expert's fragments for this wave's half of K
          // (requested and awaited by hand as well: a wait the compiler places after the branch would run in every
          // step and drain the requests of the next group)
          const bf16x8* wp = A.w1f + ((int64_t)e * KS + h * KH) * 2 * 64 + lane;
          static_for<0, KH>([&](auto ks_c) __attribute__((always_inline)) {
            constexpr int ks = decltype(ks_c)::value;
            // (the instruction's immediate offset reaches 4 KB: four fragments per base address)
            load16_async_at<((ks * 2 + 0) % 4) * 1024>(wf[ks][0], wp + ((ks * 2 + 0) / 4) * 256);
            load16_async_at<((ks * 2 + 1) % 4) * 1024>(wf[ks][1], wp + ((ks * 2 + 1) / 4) * 256);
          });
          load8_async(braw[0], A.b1s + (int64_t)e * MID_HROW + 4 * q);
          load8_async(braw[1], A.b1s + (int64_t)e * MID_HROW + 16 + 4 * q);
          asm volatile("s_waitcnt vmcnt(0)"
                       : "+v"(wf[0][0]), "+v"(wf[0][1]), "+v"(wf[1][0]), "+v"(wf[1][1]), "+v"(wf[2][0]), "+v"(wf[2][1]),
                         "+v"(wf[3][0]), "+v"(wf[3][1]), "+v"(wf[4][0]), "+v"(wf[4][1]), "+v"(wf[5][0]), "+v"(wf[5][1]),
                         "+v"(wf[6][0]), "+v"(wf[6][1]), "+v"(wf[7][0]), "+v"(wf[7][1]), "+v"(wf[8][0]), "+v"(wf[8][1]),
                         "+v"(wf[9][0]), "+v"(wf[9][1]), "+v"(wf[10][0]), "+v"(wf[10][1]), "+v"(wf[11][0]), "+v"(wf[11][1]),
                         "+v"(braw[0].x), "+v"(braw[0].y), "+v"(braw[1].x), "+v"(braw[1].y)
                       :: "memory");
          e_w = e;
        }
        f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KH; ++ks) {
          acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ks][0], xb[cur][ks], acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ks][1], xb[cur][ks], acc1, 0, 0, 0);
        }
        if (h == 1) {
          xch[pr][cur][0][lane] = acc0;
          xch[pr][cur][1][lane] = acc1;
        }
        lds_barrier();
        if (h == 0) {
          const f32x4 o0 = xch[pr][cur][0][lane], o1 = xch[pr][cur][1][lane];
          const float rw = __uint_as_float(rwb[cur] << 16);
          const int2 rec = m_rec[ph];
          const uint32_t bw[2][2] = {{(uint32_t)braw[0].x, (uint32_t)braw[0].y}, {(uint32_t)braw[1].x, (uint32_t)braw[1].y}};
          float v[8];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float bias0 = __uint_as_float((r & 1) ? (bw[0][r >> 1] & 0xffff0000u) : (bw[0][r >> 1] << 16));
            const float bias1 = __uint_as_float((r & 1) ? (bw[1][r >> 1] & 0xffff0000u) : (bw[1][r >> 1] << 16));
            const float a0 = acc0[r] + o0[r] + bias0, a1 = acc1[r] + o1[r] + bias1;
            v[r] = ((ACT >= 0) ? act_fn<ACT>(a0) : apply_act(A.act_rt, a0)) * rw;
            v[4 + r] = ((ACT >= 0) ? act_fn<ACT>(a1) : apply_act(A.act_rt, a1)) * rw;
          }
          uint2 p0, p1;
          p0.x = pack2_bf16(v[0], v[1]); p0.y = pack2_bf16(v[2], v[3]);
          p1.x = pack2_bf16(v[4], v[5]); p1.y = pack2_bf16(v[6], v[7]);
          if (q == 3) p1.y = (p1.y & 0xffffu) | ((uint32_t)(rec.x & (MID_T2 - 1)) << 16);   // element 31: row inside the tile
          if (c < m_valid[ph]) {
            bf16_t* hrow = A.hc + (int64_t)rec.y * MID_HROW + 4 * q;
            *(uint2*)hrow = p0;
            *(uint2*)(hrow + 16) = p1;
          }
        }
      }
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // requests past the end
}

// ---------------------------------------------------------------------------------------------------
// Second layer.  512 threads = 8 waves (two per SIMD); wave w owns columns [16w, 16w + 16) of the workgroup's 128.  The
// tile's hidden rows lie in memory in the order they are consumed; the work is a list of 1 KB units in LDS, per expert
// with pairs in the tile one unit "this wave's W2^T fragment of the expert" followed by its groups of 16 rows.  A wave
// keeps MID_RING units in flight.  Groups of one expert hold different tokens, and LDS executes a wave's instructions in
// order, so a later group's read of the output tile sees every earlier sum.
// ---------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(MID_DOWN_THREADS) void mid_down_kernel(const MidArgs A) {
  constexpr int NS = D / MID_DS;      // column slices
  constexpr int CT = D / 16;          // column tiles of 16
  static_assert(MID_DS / 16 == MID_DOWN_THREADS / 64, "one column tile per wave");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ int s_scan[8][2];
  __shared__ int s_tbase;
  if (A.flag[0] == 0) return;         // uniform over the grid: the dense sweep runs instead
  const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int q = lane >> 4, c = lane & 15;
  const int E = A.E;
  const int64_t N = A.N;
  // An XCD (consecutive block ids go round the XCDs) works through its tiles one column slice after the other, so the
  // W2^T fragments of the slice in hand (1 MB for 128 experts) stay in that XCD's L2.
  const int per_xcd = (A.n_tiles + 7) / 8;
  const int xcd = blockIdx.x & 7, jb = blockIdx.x >> 3;
  const int tile = (jb % per_xcd) * 8 + xcd, slice = jb / per_xcd;
  if (tile >= A.n_tiles) return;
  const int64_t tb = (int64_t)tile * MID_T2;
  const int64_t s0 = (int64_t)tile * MID_T2_SEGS, s1 = s0 + MID_T2_SEGS;
  float* ot = (float*)smem;                                  // [MID_T2 + 1][MID_OS]; the last row takes what belongs nowhere
  uint32_t* s_desc = (uint32_t*)(ot + (MID_T2 + 1) * MID_OS);
  for (int i = t; i < (MID_T2 + 1) * MID_OS / 4; i += MID_DOWN_THREADS) ((f32x4*)ot)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  // groups of the earlier tiles
  if (w == 0) {
    int tbase = 0;
    for (int i0 = 0; i0 < tile; i0 += 64) tbase += (i0 + lane < tile) ? A.tile_groups[i0 + lane] : 0;
    tbase = wave_sum_i32(tbase);
    if (lane == 0) s_tbase = tbase;
  }
  // unit list: thread e (E <= 256) owns expert e
  int cnt = 0;
  if (t < E) cnt = mid_seg_prefix(A.seg_offsets, A.totals, s1, A.n_seg, E, t) - A.seg_offsets[s0 * E + t];
  const int ng = (cnt + 15) >> 4, nu = ng ? ng + 1 : 0;
  int gi = 0, ui = 0;
  if (w < 4) {
    gi = mid_wave_incl_scan(ng, lane);
    ui = mid_wave_incl_scan(nu, lane);
    if (lane == 63) { s_scan[w][0] = gi; s_scan[w][1] = ui; }
  }
  __syncthreads();
  int gbase = 0, ubase = 0, U = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i < w) { gbase += s_scan[i][0]; ubase += s_scan[i][1]; }
    U += s_scan[i][1];
  }
  if (t < E && ng > 0) {
    const int u0 = ubase + ui - nu, g0 = gbase + gi - ng;
    s_desc[u0] = 0x80000000u | (uint32_t)t;
    for (int j = 0; j < ng; ++j) {
      const int left = cnt - 16 * j;
      s_desc[u0 + 1 + j] = (uint32_t)(g0 + j) | ((uint32_t)(left < 16 ? left : 16) << 16);
    }
  }
  __syncthreads();
  const int ct = slice * (MID_DS / 16) + w;
  if (U > 0) {
    const bf16x8* hbase = (const bf16x8*)A.hc + (int64_t)s_tbase * 64 + (c * 4 + q);   // group g of the tile: + 64 g
    const bf16x8* abase = A.w2f + (int64_t)ct * 64 + lane;                              // expert e: + e * CT * 64
    // A lane reads one descriptor per trip of MID_RING steps (units u0 + lane, the last unit again past the end); a step
    // takes its two descriptors from there with v_readlane, so no LDS read and no wait for one sits inside a step.
    auto issue = [&](bf16x8& dst, uint32_t d) __attribute__((always_inline)) {
      const bool is_a = (d & 0x80000000u) != 0u;
      const int64_t off = is_a ? (int64_t)(d & 0xffu) * (CT * 64) : (int64_t)(d & 0xffffu) * 64;
      load16_async(dst, (is_a ? abase : hbase) + off);
    };
    bf16x8 ring[MID_RING];
    uint32_t dv = s_desc[lane < U ? lane : U - 1];
    static_for<0, MID_RING - 1>([&](auto j_c) __attribute__((always_inline)) {
      issue(ring[decltype(j_c)::value], (uint32_t)__builtin_amdgcn_readlane((int)dv, decltype(j_c)::value));
    });
    bf16x8 af = {};
    f32x4 accp = {0.f, 0.f, 0.f, 0.f}, oldp = {0.f, 0.f, 0.f, 0.f};
    float* const obase = ot + w * 16 + 4 * q;
    float* addrp = obase + MID_T2 * MID_OS;                  // nothing pending: adds zeros to the spare row
    static_assert(2 * MID_RING - 1 <= 64, "a trip's descriptors fit one per lane");
    // Element 31 of row c of a group (the token's row inside the tile) sits in lane 48 + c and reaches the other lanes by
    // ds_bpermute, asked for one step ahead: it travels behind the step's read of the output tile, so the next step
    // waits once for both.
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(ring[0]) : "n"(MID_RING - 2) : "memory");
    int rb_next = __builtin_amdgcn_ds_bpermute((48 + c) * 4, (int)__builtin_bit_cast(u32x4, ring[0]).w);
    for (int u0 = 0; u0 < U; u0 += MID_RING) {
      dv = s_desc[u0 + lane < U ? u0 + lane : U - 1];
      static_for<0, MID_RING>([&](auto j_c) __attribute__((always_inline)) {
        constexpr int j = decltype(j_c)::value;
        constexpr int jn = (j + 1) % MID_RING;
        const int u = u0 + j;
        // refill the slot consumed a step ago, then wait for this step's unit and the next
        __builtin_amdgcn_sched_barrier(0);
        issue(ring[(j + MID_RING - 1) % MID_RING], (uint32_t)__builtin_amdgcn_readlane((int)dv, j + MID_RING - 1));
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(ring[j]), "+v"(ring[jn]) : "n"(MID_RING - 2) : "memory");
        const int rowbits = rb_next;
        if (u < U) {                          // uniform
          const uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)dv, j);
          if (d & 0x80000000u) {
            af = ring[j];
          } else {
            const int valid = (int)((d >> 16) & 31u);
            const u32x4 raw = __builtin_bit_cast(u32x4, ring[j]);
            const bool live = c < valid;
            const int row = live ? ((rowbits >> 16) & (MID_T2 - 1)) : MID_T2;
            u32x4 bm;
            bm.x = live ? raw.x : 0u; bm.y = live ? raw.y : 0u; bm.z = live ? raw.z : 0u; bm.w = live ? raw.w : 0u;
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            const f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8, bm), z, 0, 0, 0);
            float* const addr = obase + row * MID_OS;
            // finish the group before: its sums, then this group's read (behind the write: the rows may coincide)
            *(f32x4*)addrp = oldp + accp;
            oldp = *(const f32x4*)addr;
            accp = acc;
            addrp = addr;
          }
        }
        rb_next = __builtin_amdgcn_ds_bpermute((48 + c) * 4, (int)__builtin_bit_cast(u32x4, ring[jn]).w);
      });
    }
    *(f32x4*)addrp = oldp + accp;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the refills past the end
  }
  __syncthreads();

  // rows leave as bf16 after + last_bias (+ x): 16 threads per row, 8 columns each
  const int live = (int)((N - tb) < (int64_t)MID_T2 ? (N - tb) : (int64_t)MID_T2);
  const int c8 = (t & 15) * 8;
  const int col = slice * MID_DS + c8;
  float lb[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) lb[i] = (A.last_bias != nullptr) ? bf16_to_f32(A.last_bias[col + i]) : 0.f;
  for (int r = t >> 4; r < live; r += MID_DOWN_THREADS / 16) {
    const f32x4 a0 = *(const f32x4*)(ot + r * MID_OS + c8), a1 = *(const f32x4*)(ot + r * MID_OS + c8 + 4);
    float v[8] = {a0[0] + lb[0], a0[1] + lb[1], a0[2] + lb[2], a0[3] + lb[3], a1[0] + lb[4], a1[1] + lb[5], a1[2] + lb[6], a1[3] + lb[7]};
    if (A.add_residual) {
      const u32x4 xr = *(const u32x4*)(A.x + (tb + r) * D + col);
      const uint32_t xw[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] += __uint_as_float((i & 1) ? (xw[i >> 1] & 0xffff0000u) : (xw[i >> 1] << 16));
    }
    u32x4 o;
    o.x = pack2_bf16(v[0], v[1]); o.y = pack2_bf16(v[2], v[3]); o.z = pack2_bf16(v[4], v[5]); o.w = pack2_bf16(v[6], v[7]);
    *(u32x4*)(A.out + (tb + r) * D + col) = o;
  }
}

template <int ACT>
static hipError_t launch_mid_up(const MidArgs& A, unsigned grid, hipStream_t s) {
  hipLaunchKernelGGL((mid_up_kernel<768, ACT>), dim3(grid), dim3(MID_UP_THREADS), 0, s, A);
  return hipGetLastError();
}

// Plans the call on the device, runs the two kernels when the routed pairs fit the provisioned capacity, and leaves
// *flag == 0 otherwise so that the dense sweep (launched by the caller with skip_flag = the returned pointer) does the work.
hipError_t launch_mfma_mid(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                           const void* last_bias, void* out, void* workspace, const int** flag_out, hipStream_t s) {
  const MidWorkspace W = mid_workspace(sh);
  const PackedLayout L = packed_layout(sh);
  char* ws = (char*)workspace;
  const char* pk = (const char*)packed;
  const int64_t N = sh.n_tokens;
  const int E = sh.n_experts;
  const int cus = device_cu_count();
  MidArgs A;
  A.x = (const bf16_t*)x; A.routing = (const bf16_t*)routing;
  A.w1f = (const bf16x8*)(pk + L.m1_off); A.w2f = (const bf16x8*)(pk + L.m2_off); A.b1s = (const bf16_t*)(pk + L.sb_off);
  A.seg_offsets = (const int32_t*)(ws + W.seg_offsets); A.totals = (const int32_t*)(ws + W.totals);
  A.offsets = (int32_t*)(ws + W.offsets); A.flag = (int32_t*)(ws + W.flag); A.tile_groups = (int32_t*)(ws + W.tile_groups);
  A.rec = (int2*)(ws + W.rec); A.hc = (bf16_t*)(ws + W.hc); A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out;
  A.N = N; A.cap = W.cap; A.E = E; A.n_seg = (int)W.n_seg; A.n_tiles = (int)W.n_tiles; A.act_rt = sh.activation;
  A.add_residual = sh.add_residual;
  launch_plan_count_scan(routing, N, E, (int32_t*)(ws + W.seg_counts), (int32_t*)(ws + W.seg_pairs),
                         (int32_t*)(ws + W.seg_offsets), (int32_t*)(ws + W.totals), s);
  hipLaunchKernelGGL(mid_tile_kernel, dim3((unsigned)cdiv64(W.n_tiles, 4)), dim3(256), 0, s, A.seg_offsets, A.totals,
                     A.tile_groups, E, A.n_seg, A.n_tiles);
  const unsigned seg_blocks = (unsigned)cdiv64(W.n_seg, 4);
  const int vpt = (E + 63) / 64;
#define D2DMOE_MID_SCATTER(V)                                                                                            \
  hipLaunchKernelGGL(mid_scatter_kernel<V>, dim3(seg_blocks), dim3(256), 0, s, A.routing, A.seg_offsets, A.totals,       \
                     A.tile_groups, A.offsets, A.flag, A.rec, N, E, A.n_seg, W.cap)
  if (vpt <= 1) D2DMOE_MID_SCATTER(1); else if (vpt <= 2) D2DMOE_MID_SCATTER(2); else D2DMOE_MID_SCATTER(4);
#undef D2DMOE_MID_SCATTER
  hipError_t e;
  const unsigned grid1 = (unsigned)cus;
  switch (sh.activation) {
    case D2DMOE_ACT_RELU: e = launch_mid_up<D2DMOE_ACT_RELU>(A, grid1, s); break;
    case D2DMOE_ACT_GELU: e = launch_mid_up<D2DMOE_ACT_GELU>(A, grid1, s); break;
    default: e = launch_mid_up<-1>(A, grid1, s); break;
  }
  if (e != hipSuccess) return e;
  // output tile + spare row, unit list: an expert unit and up to 16 groups per expert
  const size_t lds2 = (size_t)(MID_T2 + 1) * MID_OS * 4 + (size_t)E * (MID_T2 / 16 + 1) * 4;
  e = hipFuncSetAttribute((const void*)mid_down_kernel<768>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2);
  if (e != hipSuccess) return e;
  const unsigned grid2 = (unsigned)(8 * cdiv64(W.n_tiles, 8) * (sh.d_model / MID_DS));
  hipLaunchKernelGGL((mid_down_kernel<768>), dim3(grid2), dim3(MID_DOWN_THREADS), lds2, s, A);
  *flag_out = A.flag;
  return hipGetLastError();
}

}  // namespace d2dmoe
