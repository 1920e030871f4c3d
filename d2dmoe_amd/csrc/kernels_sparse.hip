// Expert-major bf16 MFMA path for sparse routing (few experts per token): device-side plan (permutation, tiles,
// path flag), grouped per-expert fused up-projection + activation + down-projection, and the ordered combine.
//
//   plan     routing [N,E]  ->  offsets[E+1], token_idx[P] (expert-major, tokens ascending: the canonical permutation),
//                               tok_off[N+1] (token-major offsets), pair_dst[P] (expert-major pair -> token-major
//                               slot, experts ascending inside a token), tile_off[E+1] (tiles of 32 pairs), flag
//   experts  a workgroup per group of up to 8 tiles of 32 (token, expert) pairs of ONE expert, whose weights stay in
//            registers while the tiles pass: gather a tile's 32 x rows, GEMM1 against the expert's W1 fragments, bias
//            + activation + routing weight, GEMM2 against its W2^T fragments, store the 32 result rows (16-bit, as the
//            reference's per-expert intermediate is) at their token-major slots
//   combine  out[n] = sum over the token's slots in ascending expert order, float32, one rounding, + last_bias (+ x)
//            -- the order of the reference's merge kernel (moe_impls.py:499-514), no atomics.
// Nothing is decided on the host: when the routed pairs exceed the provisioned capacity the flag stays 0, these
// kernels return at once and the dense sweep (launched after them with the same flag) does the work.
#include "mfma_common.hpp"

namespace d2dmoe {

constexpr int SP_BT = 32;        // pairs per tile

struct SparseWorkspace {
  int64_t n_seg, cap;
  size_t seg_counts, seg_offsets, totals, seg_pairs, offsets, tile_off, flag, tok_off, token_idx, pair_dst, y,
      total;
};

// Routed pairs per token the path is provisioned for.  Ungated experts (36 KB each at the ViT-B shape): 8 -- the dense
// sweep is as fast from about 8 on.  Gated experts at the Gemma shape (786 KB each): the tiled products cost 0.8 ms per
// 4096 tokens whatever the routing and the expert-major kernels stay below that up to about 40 pairs per token, so the
// capacity is 32 -- up to 16 384 tokens, where the per-pair rows (4 KB each) take 2 GB; beyond that 8.
int mfma_sparse_capacity_k(const d2dmoe_shape& sh) {
  if (sh.gated) return (sh.n_tokens <= 16384) ? SP_MAX_MEAN_K_GATED : SP_MAX_MEAN_K;
  // D = 1024 / 1280: the alternative is the tiled products (1.3 ms at 50 432 tokens, 128 experts x 32, against 0.15 ms +
  // 0.07 ms per routed expert per token here)
  if (sh.d_model != 768) return sh.expert_dim <= 32 ? 12 : 6;
  return SP_MAX_MEAN_K;   // ~45 us + 40 - 52 us per routed expert per token against 0.44 - 0.49 ms for the sweep
}

static SparseWorkspace sparse_workspace(const d2dmoe_shape& sh, int max_mean_k) {
  SparseWorkspace W;
  const int64_t N = sh.n_tokens;
  const int E = sh.n_experts;
  W.n_seg = cdiv64(N, SP_SEG);
  W.cap = N * max_mean_k;
  // Gated experts, few tokens: whatever the routing, an expert's 786 KB of weights are streamed once or twice, so the
  // path also pays with every expert routed to by every token -- room for at least 128 pairs per expert.
  if (sh.gated && N > 16 && W.cap < (int64_t)E * SP_GATED_MIN_PAIRS_PER_EXPERT) W.cap = (int64_t)E * SP_GATED_MIN_PAIRS_PER_EXPERT;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += (bytes + 255) / 256 * 256; return o; };
  W.seg_counts = take((size_t)W.n_seg * E * 4);
  W.seg_offsets = take((size_t)W.n_seg * E * 4);
  W.totals = take((size_t)E * 4);
  W.seg_pairs = take((size_t)W.n_seg * 4);
  W.offsets = take((size_t)(E + 1) * 4);
  W.tile_off = take((size_t)(E + 1) * 4);
  W.flag = take(16);
  W.tok_off = take((size_t)(N + 1) * 4);
  W.token_idx = take((size_t)W.cap * 4);
  W.pair_dst = take((size_t)W.cap * 4);
  size_t ybytes = (size_t)W.cap * sh.d_model * 2;
  if (!mfma_sparse_falls_back_to_sweep(sh)) {   // where the fall-back is the tiled products, they work in the same region
    const size_t g = mfma_gemm_workspace_bytes(sh);
    if (g > ybytes) ybytes = g;
  }
  W.y = take(ybytes);
  W.total = off;
  return W;
}

int64_t mfma_sparse_capacity_pairs(const d2dmoe_shape& sh) { return sparse_workspace(sh, mfma_sparse_capacity_k(sh)).cap; }

size_t mfma_sparse_fallback_offset(const d2dmoe_shape& sh) { return sparse_workspace(sh, mfma_sparse_capacity_k(sh)).y; }

size_t mfma_sparse_workspace_bytes(const d2dmoe_shape& sh) {
  if (!mfma_sparse_supported(sh)) return 0;
  return sparse_workspace(sh, mfma_sparse_capacity_k(sh)).total;
}

// ---------------------------------------------------------------------------------------------------
// Packing of the expert-major section.  nt = row tiles of 32 neurons per expert (Ed padded to nt*32 with zeros).
//   W1 fragments   [E][kstep D/16][nt][lane][8]:  neuron j = t*32 + c, d = kstep*16 + 8g + i          w1[e][d][j]
//   W2^T fragments [E][col-tile D/32][kstep2 2 nt][lane][8]:  column = ct*32 + c,
//                  neuron j = (ks2/2)*32 + (ks2%2)*16 + 8*(i/4) + 4g + (i%4)                           w2[e][j][column]
//   bias           [E][nt*32] bf16
// ---------------------------------------------------------------------------------------------------
__global__ void pack_sparse_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ b1, const bf16_t* __restrict__ w2,
                                   bf16_t* __restrict__ d1, bf16_t* __restrict__ d2, bf16_t* __restrict__ db, int D, int E,
                                   int Ed, int nt) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per_expert = (int64_t)nt * 32 * D / 8;   // 16-byte pieces per expert in either fragment array
  const int64_t n = (int64_t)E * per_expert;
  const int lane = (int)(p % 64);
  const int g = lane / 32, c = lane % 32;
  if (p < n) {
    if (w1 == nullptr) return;
    const int e = (int)(p / per_expert);
    int64_t q = (p % per_expert) / 64;
    const int t = (int)(q % nt);
    const int ks = (int)(q / nt);
    const int j = t * 32 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 16 + 8 * g + i;
      d1[p * 8 + i] = (j < Ed) ? w1[((int64_t)e * D + d) * Ed + j] : (bf16_t)0;
    }
  } else if (p < 2 * n) {
    if (w2 == nullptr) return;
    const int64_t pp = p - n;
    const int e = (int)(pp / per_expert);
    int64_t q = (pp % per_expert) / 64;
    const int ks2 = (int)(q % (2 * nt));
    const int ct = (int)(q / (2 * nt));
    const int col = ct * 32 + c;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = (ks2 / 2) * 32 + (ks2 % 2) * 16 + 8 * (i / 4) + 4 * g + (i % 4);
      d2[pp * 8 + i] = (j < Ed) ? w2[((int64_t)e * Ed + j) * D + col] : (bf16_t)0;
    }
  } else if (p < 2 * n + (int64_t)E * nt * 32) {
    if (db == nullptr) return;
    const int64_t pp = p - 2 * n;
    const int e = (int)(pp / (nt * 32)), j = (int)(pp % (nt * 32));
    db[pp] = (j < Ed && b1 != nullptr) ? b1[(int64_t)e * Ed + j] : (bf16_t)0;
  }
}

hipError_t launch_sparse_pack(const d2dmoe_shape& sh, const PackedLayout& L, const void* w1, const void* b1, const void* w2,
                              const void* w_up, void* packed, hipStream_t s) {
  char* base = (char*)packed;
  const int64_t n = 2 * (int64_t)sh.n_experts * L.nt * 32 * sh.d_model / 8 + (int64_t)sh.n_experts * L.nt * 32;
  if (sh.gated) {
    // gated experts: the up projection is a second stream in the W1 arrangement; there is no bias
    hipLaunchKernelGGL(pack_sparse_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)w_up,
                       (const bf16_t*)nullptr, (const bf16_t*)nullptr, (bf16_t*)(base + L.su_off), (bf16_t*)nullptr,
                       (bf16_t*)nullptr, sh.d_model, sh.n_experts, sh.expert_dim, L.nt);
  }
  hipLaunchKernelGGL(pack_sparse_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)w1,
                     (const bf16_t*)b1, (const bf16_t*)w2, (bf16_t*)(base + L.s1_off), (bf16_t*)(base + L.s2_off),
                     (bf16_t*)(base + L.sb_off), sh.d_model, sh.n_experts, sh.expert_dim, L.nt);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------
// Plan, pass 1: per segment of SP_SEG tokens (one wave, lanes = experts) the number of routed tokens per expert and the
// segment's number of pairs.
// ---------------------------------------------------------------------------------------------------
template <int VPT>
__global__ __launch_bounds__(256) void plan_count_kernel(const bf16_t* __restrict__ routing, int32_t* __restrict__ seg_counts,
                                                         int32_t* __restrict__ seg_pairs, int64_t N, int E, int64_t n_seg) {
  const int lane = threadIdx.x & 63;
  const int64_t seg = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / 64;
  if (seg >= n_seg) return;
  const int vpt = (E + 63) / 64;
  const int64_t t0 = seg * SP_SEG;
  const int rows = (int)((N - t0) < SP_SEG ? (N - t0) : SP_SEG);
  int cnt[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) cnt[k] = 0;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    if (k < vpt) {   // uniform
      const int e = lane + k * 64;
      bf16_t v[SP_SEG];   // the segment's rows for this lane group, fetched together
#pragma unroll
      for (int i = 0; i < SP_SEG; ++i) {
        const int r = (i < rows) ? i : (rows - 1);
        v[i] = routing[(t0 + r) * E + (e < E ? e : E - 1)];   // unconditional (clamped): the loads go out together
      }
#pragma unroll
      for (int i = 0; i < SP_SEG; ++i)
        if (i < rows && e < E) cnt[k] += ((v[i] & 0x7fff) != 0) ? 1 : 0;   // non-zero routing weight
    }
  }
  int tot = 0;
#pragma unroll
  for (int k = 0; k < VPT; ++k)
    if (k < vpt) {
      const int e = lane + k * 64;
      if (e < E) seg_counts[seg * E + e] = cnt[k];
      tot += cnt[k];
    }
  tot = wave_sum_i32(tot);
  if (lane == 0) seg_pairs[seg] = tot;
}

// Plan, pass 3 (after the per-expert scan over segments): scatter.  A wave walks its segment's tokens in order;
// lanes = experts, so a lane's running counter is the token's rank inside the expert's list (expert-major position)
// and a prefix count over the lanes is the expert's rank inside the token's list (token-major position).
// What a wave needs of the global picture it derives itself from the small arrays of the earlier passes: the experts'
// offsets (a scan over E totals), its segment's first token-major slot (a sum over the segments before it) and the
// path flag (all pairs <= capacity).  The first wave also publishes offsets, tile offsets, the flag and tok_off[N]
// for the kernels that follow, so no single-workgroup pass sits between the scan and this one.
// ---------------------------------------------------------------------------------------------------
__device__ inline int wave_incl_scan_i32(int v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int t = __shfl_up(v, off, 64);
    if (lane >= off) v += t;
  }
  return v;
}

template <int VPT>
__global__ __launch_bounds__(256) void plan_scatter_kernel(const bf16_t* __restrict__ routing, const int32_t* __restrict__ seg_offsets,
                                                           const int32_t* __restrict__ totals, const int32_t* __restrict__ seg_pairs,
                                                           int32_t* __restrict__ offsets, int32_t* __restrict__ tile_off,
                                                           int32_t* __restrict__ flag, int32_t* __restrict__ tok_off,
                                                           int32_t* __restrict__ token_idx, int32_t* __restrict__ pair_dst,
                                                           int64_t N, int E, int64_t n_seg, int64_t cap, int split) {
  // split == 0: a wave per segment, four segments per workgroup.  split != 0 (few segments): a workgroup per segment,
  // whose four waves each scatter a quarter of the segment's tokens (the per-token loop is the serial part of this
  // kernel) after the same prologue: where a wave's first token starts follows from the bits of the tokens before it.
  const int lane = threadIdx.x & 63, wq = threadIdx.x >> 6;
  const int64_t seg = split ? (int64_t)blockIdx.x : ((int64_t)blockIdx.x * 4 + wq);
  if (seg >= n_seg) return;
  const int vpt = (E + 63) / 64;
  const int64_t t0 = seg * SP_SEG;
  const int rows = (int)((N - t0) < SP_SEG ? (N - t0) : SP_SEG);
  constexpr int RPW = SP_SEG / 4;                 // tokens per wave when the segment is split
  const int row_lo = split ? wq * RPW : 0;
  const int row_hi = split ? ((row_lo + RPW < rows) ? (row_lo + RPW) : rows) : rows;
  const bool first_wave = (seg == 0) && (split ? wq == 0 : true);
  // Every load of the prologue is issued before anything is computed from it, none of them under a branch (lane
  // groups past the last expert read clamped addresses and are masked), so the wave pays about one round trip.
  int tot[VPT], segoff[VPT];
  unsigned onbits[VPT];    // bit i = token i of the segment routes to expert e
  static_assert(SP_SEG <= 32, "one 32-bit mask per lane group");
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int e = lane + k * 64;
    const int ec = (e < E) ? e : (E - 1);
    tot[k] = totals[ec];
    segoff[k] = seg_offsets[seg * E + ec];
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
  // pairs of all earlier segments = this segment's first token-major slot; eight loads per trip
  int before_segs = 0;
  for (int64_t s0 = 0; s0 < seg; s0 += 512) {
    int part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t sgi = s0 + u * 64 + lane;
      part[u] = seg_pairs[sgi < seg ? sgi : 0];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) before_segs += (s0 + u * 64 + lane < seg) ? part[u] : 0;
  }
  before_segs = wave_sum_i32(before_segs);
  // exclusive scans over the experts (e = lane + 64 k) of the pair counts and of the tile counts
  int eoff[VPT], toff[VPT];
  int run = 0, trun = 0;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int e = lane + k * 64;
    const int c = (e < E) ? tot[k] : 0;
    const int tc = (c + SP_BT - 1) / SP_BT;
    const int ci = wave_incl_scan_i32(c, lane), ti = wave_incl_scan_i32(tc, lane);
    eoff[k] = run + ci - c;
    toff[k] = trun + ti - tc;
    run += __shfl(ci, 63, 64);
    trun += __shfl(ti, 63, 64);
  }
  const int64_t P = run;
  const bool sparse_ok = P <= cap;
  if (first_wave) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int e = lane + k * 64;
      if (e < E) {
        offsets[e] = eoff[k];
        tile_off[e] = toff[k];
      }
    }
    if (lane == 0) {
      offsets[E] = run;
      tile_off[E] = trun;
      flag[0] = sparse_ok ? 1 : 0;
      tok_off[N] = (int32_t)P;
    }
  }
  if (!sparse_ok) return;
  int pos[VPT];            // next expert-major position of expert e
  const unsigned below = (row_lo == 0) ? 0u : ((1u << row_lo) - 1u);   // the segment's tokens before this wave's
  int earlier = 0;         // their pairs
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int c = __popc(onbits[k] & below);
    pos[k] = eoff[k] + segoff[k] + c;
    earlier += c;
  }
  int tokbase = before_segs + wave_sum_i32(earlier);
  const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int i = row_lo; i < row_hi; ++i) {
    const int64_t tok = t0 + i;
    int before = 0;   // routed experts of this token with a smaller index, over the previous lane groups
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      if (k < vpt) {
        const bool on = ((onbits[k] >> i) & 1u) != 0u;
        const unsigned long long bal = __ballot(on);
        if (on) {
          const int rank_in_token = before + __popcll(bal & lt_mask);
          token_idx[pos[k]] = (int32_t)tok;
          pair_dst[pos[k]] = tokbase + rank_in_token;
          pos[k] += 1;
        }
        before += __popcll(bal);
      }
    }
    if (lane == 0) tok_off[tok] = tokbase;
    tokbase += before;
  }
}

// Arguments of the expert-major experts kernels.
struct SparseArgs {
  const bf16_t* x; const bf16_t* routing; const bf16x8* w1s; const bf16x8* w2s; const bf16_t* b1s;
  const bf16x8* wus;   // gated experts: fragments of the up projection, arranged like w1s
  const int32_t* offsets; const int32_t* tile_off; const int32_t* token_idx; const int32_t* pair_dst; const int32_t* flag;
  bf16_t* y; int E; int act_rt;
  const int32_t* tok_off; const bf16_t* last_bias; bf16_t* out; int add_residual;   // tokens with ONE routed expert
};

// ---------------------------------------------------------------------------------------------------
// Expert-major fused experts kernel.  256 threads = 4 waves; a workgroup takes a GROUP of up to SG_MAX tiles of 32
// pairs of one expert and keeps the expert's weights in registers while the tiles pass -- W1 (this wave's quarter of
// the model dimension, NT row tiles of 32 neurons) through the first product of every tile of the group, then W2^T
// (this wave's quarter of the output columns) in the same registers through the second product of every tile.  (With
// one tile per weight load an expert of 128 neurons costs 12 KB of weight traffic per pair; here 1.5 - 3 KB.)
//   First product (transposed, H^T = W1^T . X^T), split over K: wave w multiplies its quarter of the model dimension,
//   reading the x rows straight from their gathered positions as B fragments, one tile ahead; the four partial tiles
//   are summed through LDS in wave order.  Wave w finishes accumulator quad w of every row tile -- bias, activation,
//   routing weight, rounding to 16 bits -- and leaves the values in LDS in B-fragment position for the second product.
//   Second product (also transposed: OUT^T = W2^T . H^T), K outside so that D / 128 accumulators sit between
//   dependent MFMAs.  A lane ends with ONE pair and 4 consecutive columns per accumulator quad; rows leave through the
//   wave's slice of the partial-sum buffer, two column tiles at a time, so that 8 lanes write 128 contiguous bytes of
//   a row: into the pair's token-major slot of y, or, for a token with a single routed expert, finished
//   (+ last_bias (+ x), one rounding) into out.
// The group size is chosen per launch from the number of tiles (whole rounds over the grid, overhead per group), the
// same value in every workgroup; the expert of a group is found by bisection over the groups-per-expert prefix sums.
// ---------------------------------------------------------------------------------------------------
constexpr int SG_MAX = 8;
// workgroups per CU: the weights a wave keeps (D / 64 * NT fragments) and its output accumulators (D / 8 registers)
// leave room for two at D = 768 with one or two row tiles and at D = 1024 with one
constexpr int sg_wgs_per_cu(int D, int NT) { return (D <= 1024 && D * NT <= 1536) ? 2 : 1; }
template <int NT> constexpr size_t sg_lds_bytes(int D) {
  return (size_t)4 * NT * 16 * 64 * 4 + (size_t)SG_MAX * 2 * NT * 64 * 16 + (size_t)2 * 1025 * 4 + (size_t)4 * SG_MAX * 32 * 4 + (size_t)D * 2;
}

template <int D, int NT, int ACT, bool F16 = false>
__global__ __launch_bounds__(256, sg_wgs_per_cu(D, NT)) void experts_mfma_group_kernel(const SparseArgs A) {
  constexpr int KS1 = D / 16;
  constexpr int KQ = KS1 / 4;    // K steps per wave
  constexpr int CTW = D / 128;   // column tiles per wave
  static_assert(KS1 % 4 == 0 && CTW % 2 == 0, "the model dimension must split over four waves");
  extern __shared__ __attribute__((aligned(16))) unsigned char sg_smem[];
  typedef float PartT[NT * 16][64];
  PartT* part = (PartT*)sg_smem;                                     // [4][NT*16][64]
  uint4* hbs = (uint4*)(sg_smem + (size_t)4 * NT * 16 * 64 * 4);     // [SG_MAX][2 NT][64]: hidden values, B fragments
  int32_t* s_goff = (int32_t*)(hbs + SG_MAX * 2 * NT * 64);          // [1025] groups before expert e
  int32_t* s_offsets = s_goff + 1025;                                // [1025]
  int32_t* s_tok = s_offsets + 1025;                                 // [SG_MAX][32] the group's pairs: token,
  int32_t* s_dst = s_tok + SG_MAX * 32;                              //   row of y,
  float* s_rw = (float*)(s_dst + SG_MAX * 32);                       //   routing weight,
  int32_t* s_single = (int32_t*)(s_rw + SG_MAX * 32);                //   whether it is its token's only pair
  bf16_t* s_last_bias = (bf16_t*)(s_single + SG_MAX * 32);           // [D]
  if (A.flag[0] == 0) return;
  const int E = A.E;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = lane >> 5, c32 = lane & 31;
  for (int i = threadIdx.x; i <= E; i += 256) s_offsets[i] = A.offsets[i];
  for (int i = threadIdx.x; i < D; i += 256) s_last_bias[i] = (A.last_bias != nullptr) ? A.last_bias[i] : (bf16_t)0;
  // group size: whole rounds over the grid cost (tiles per group + about 3 tile times of weight loads and waits) each
  const int n_tiles = A.tile_off[E];
  int gs = 1;
  {
    int64_t best = -1;
    for (int c = 1; c <= SG_MAX; ++c) {
      const int groups = (n_tiles + c - 1) / c + E / 2;
      const int64_t cost = (int64_t)((groups + (int)gridDim.x - 1) / (int)gridDim.x) * (c + 3);
      if (best < 0 || cost <= best) { best = cost; gs = c; }
    }
  }
  __syncthreads();
  if (w == 0) {   // groups before each expert: inclusive scan, 64 experts at a time
    int carry = 0;
    for (int b = 0; b < E; b += 64) {
      const int e = b + lane;
      int v = 0;
      if (e < E) {
        const int tiles = (s_offsets[e + 1] - s_offsets[e] + SP_BT - 1) / SP_BT;
        v = (tiles + gs - 1) / gs;
      }
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(v, d, kWave);
        if (lane >= d) v += o;
      }
      if (e < E) s_goff[e + 1] = carry + v;
      carry += __shfl(v, 63, kWave);
    }
    if (lane == 0) s_goff[0] = 0;
  }
  __syncthreads();
  const int n_groups = s_goff[E];

  for (int G = blockIdx.x; G < n_groups; G += gridDim.x) {
    int lo = 0, hi = E;   // largest e with goff[e] <= G (experts without groups share their successor's offset)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_goff[mid] <= G) lo = mid; else hi = mid;
    }
    const int e = lo;
    const int base = s_offsets[e] + (G - s_goff[e]) * gs * SP_BT;
    int np = s_offsets[e + 1] - base;
    if (np > gs * SP_BT) np = gs * SP_BT;
    const int nsub = (np + SP_BT - 1) / SP_BT;

    // W1 fragments of this wave's quarter of K: requested first, the pairs' records travel at the same time
    const bf16x8* w1f = A.w1s + ((int64_t)e * KS1 + w * KQ) * NT * 64 + lane;
    bf16x8 wr[KQ * NT];
    static_assert(KQ * NT == CTW * 2 * NT, "both weight sets fill the same registers");
#pragma unroll
    for (int i = 0; i < KQ * NT; ++i) wr[i] = w1f[i * 64];
    {
      const int j = threadIdx.x;             // pair j of the group (sub-tile j / 32); short sub-tiles repeat their last pair
      const int jj = (j < np) ? j : (((j >> 5) < nsub) ? np - 1 : 0);
      if ((j >> 5) < nsub) {
        const int tok = A.token_idx[base + jj];
        s_tok[j] = tok;
        s_dst[j] = A.pair_dst[base + jj];
        s_single[j] = (A.tok_off[tok + 1] - A.tok_off[tok] == 1) ? 1 : 0;
        s_rw[j] = dec16<F16>(A.routing[(int64_t)tok * E + e]);
      }
    }
    __syncthreads();

    // ---- first product of every tile of the group
    const bf16_t* bias_e = A.b1s + (int64_t)e * NT * 32;
    uint2 bqr[NT];   // biases of the rows this wave finishes (quad w of every row tile): fetched once per group
#pragma unroll
    for (int t = 0; t < NT; ++t) bqr[t] = *(const uint2*)(bias_e + t * 32 + 8 * w + 4 * g);
    // x rows are requested one tile ahead, into the set of registers the tile after this one computes from (two sets
    // that swap roles: a copy at the end of the trip would be scheduled right behind each last use and wait for the
    // read-ahead there).  At three workgroups per CU, where a second set does not fit, the kernel spills and runs
    // slower than at two.
    bf16x8 x0[KQ], x1[KQ];
    {
      const bf16x8* xrow = (const bf16x8*)(A.x + (int64_t)s_tok[c32] * D) + 2 * w * KQ + g;
#pragma unroll
      for (int ks = 0; ks < KQ; ++ks) x0[ks] = xrow[2 * ks];
    }
    // Everything requested so far (weights, the first tile's x rows) is waited for HERE: a wait left to the loop body
    // would, from the second trip on, count the rows requested at the top of the trip instead.
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
    auto first_product = [&](const int sb, bf16x8 (&xc)[KQ], bf16x8 (&xn)[KQ]) __attribute__((always_inline)) {
      {   // the next tile's x rows (the last trip re-reads its own)
        const int sn = (sb + 1 < nsub) ? sb + 1 : sb;
        const bf16x8* xrow = (const bf16x8*)(A.x + (int64_t)s_tok[sn * 32 + c32] * D) + 2 * w * KQ + g;
#pragma unroll
        for (int ks = 0; ks < KQ; ++ks) xn[ks] = xrow[2 * ks];
      }
      f32x16 acc1[NT];
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc1[a][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KQ; ++ks)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc1[t] = mfma_32x32x16<F16>(wr[ks * NT + t], xc[ks], acc1[t]);
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) part[w][t * 16 + r][lane] = acc1[t][r];
      __syncthreads();
      const float rw = s_rw[sb * 32 + c32];
      // wave w finishes accumulator quad w (4 neurons per lane) of every row tile: 8 bytes of a B fragment each
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint2 bq = bqr[t];
        const float bias[4] = {dec16<F16>(bq.x & 0xffffu), dec16_hi<F16>(bq.x), dec16<F16>(bq.y & 0xffffu), dec16_hi<F16>(bq.y)};
        float hv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = w * 4 + i;
          float v = ((part[0][t * 16 + r][lane] + part[1][t * 16 + r][lane]) + part[2][t * 16 + r][lane]) +
                    part[3][t * 16 + r][lane];
          v += bias[i];
          v = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(A.act_rt, v);
          hv[i] = v * rw;
        }
        uint2 pk;
        pk.x = enc16x2<F16>(hv[0], hv[1]);
        pk.y = enc16x2<F16>(hv[2], hv[3]);
        ((uint2*)(hbs + (sb * 2 * NT + t * 2 + (w >> 1)) * 64 + lane))[w & 1] = pk;
      }
      __syncthreads();   // partial tiles are rewritten by the next tile; the hidden fragments are complete
    };
    for (int sb = 0; sb < nsub; sb += 2) {
      first_product(sb, x0, x1);
      if (sb + 1 < nsub) first_product(sb + 1, x1, x0);
    }

    // ---- second product of every tile of the group: W2^T fragments of this wave's columns take the registers over
    const bf16x8* w2f = A.w2s + ((int64_t)e * (D / 32) + w * CTW) * (2 * NT) * 64 + lane;
#pragma unroll
    for (int i = 0; i < CTW * 2 * NT; ++i) wr[i] = w2f[i * 64];
    const int col0 = w * (D / 4) + 4 * g;
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): the weights; inside the loop the count would be the previous tile's row stores
    for (int sb = 0; sb < nsub; ++sb) {
      const int rows = (np - sb * SP_BT < SP_BT) ? (np - sb * SP_BT) : SP_BT;
      const int tok = s_tok[sb * 32 + c32], dst = s_dst[sb * 32 + c32];
      const bool single = (c32 < rows) && s_single[sb * 32 + c32] != 0;
      bf16x8 hb[2 * NT];
#pragma unroll
      for (int k2 = 0; k2 < 2 * NT; ++k2) {
        const uint4 v = hbs[(sb * 2 * NT + k2) * 64 + lane];
        __builtin_memcpy(&hb[k2], &v, 16);
      }
      f32x16 acc2[CTW];
#pragma unroll
      for (int a = 0; a < CTW; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[a][r] = 0.f;
#pragma unroll
      for (int ks2 = 0; ks2 < 2 * NT; ++ks2) {   // K outside: CTW independent accumulators between dependent MFMAs
#pragma unroll
        for (int ct = 0; ct < CTW; ++ct) acc2[ct] = mfma_32x32x16<F16>(wr[ct * 2 * NT + ks2], hb[ks2], acc2[ct]);
        __builtin_amdgcn_sched_barrier(0);
      }
      const bool any_single = __ballot(single) != 0ull;   // uniform
      if (any_single) {
        const uint32_t keep = single ? 0xffffffffu : 0u;
        const bf16_t* xres = A.x + (int64_t)tok * D + col0;
        // + last_bias on the rows of those pairs, by the matrix unit: one more K step whose only non-zero entries are
        // the bias (k = 0 of the column's A fragment) and 1.0 for such a pair (k = 0 of its B fragment) -- an exact product,
        // added to the accumulator with the one rounding a float addition has.  (A bias that is not finite would spread to
        // the other pairs' rows as NaN; their tokens' results carry that bias anyway.)
        {
          const uint32_t one16 = F16 ? 0x3c00u : 0x3f80u;
          const u32x4 kb = {(g == 0 && single) ? one16 : 0u, 0u, 0u, 0u};
          bf16x8 keep_b;
          __builtin_memcpy(&keep_b, &kb, 16);
          uint32_t lbv[CTW];
#pragma unroll
          for (int ct = 0; ct < CTW; ++ct) lbv[ct] = s_last_bias[w * (D / 4) + ct * 32 + c32];
#pragma unroll
          for (int ct = 0; ct < CTW; ++ct) {
            const u32x4 ab = {(g == 0) ? lbv[ct] : 0u, 0u, 0u, 0u};
            bf16x8 bias_a;
            __builtin_memcpy(&bias_a, &ab, 16);
            acc2[ct] = mfma_32x32x16<F16>(bias_a, keep_b, acc2[ct]);
          }
        }
        if (A.add_residual) {   // uniform; after the bias, as in the combine kernel
#pragma unroll
          for (int ct = 0; ct < CTW; ++ct) {
            uint2 xv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) xv[q] = *(const uint2*)(xres + ct * 32 + 8 * q);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint32_t vx = xv[q].x & keep, vy = xv[q].y & keep;
              acc2[ct][q * 4 + 0] += dec16<F16>(vx & 0xffffu);
              acc2[ct][q * 4 + 1] += dec16_hi<F16>(vx);
              acc2[ct][q * 4 + 2] += dec16<F16>(vy & 0xffffu);
              acc2[ct][q * 4 + 3] += dec16_hi<F16>(vy);
            }
          }
        }
      }
      // rows leave through this wave's slice of the partial-sum buffer (no other wave touches it in this phase)
      {
        unsigned char* stage = (unsigned char*)&part[w][0][0];   // 32 rows x 128 bytes
        const int ridx = single ? tok : dst;
        const int rl = lane >> 3, pc = lane & 7;
        bf16_t* rptr[4];
        bool rlive[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int R = rl + 8 * i;
          const int idx = __shfl(ridx, R, kWave);
          const int sg = __shfl((int)single, R, kWave);
          rptr[i] = (sg ? A.out : A.y) + (int64_t)idx * D + w * (D / 4) + pc * 8;
          rlive[i] = R < rows;
        }
#pragma unroll
        for (int ps = 0; ps < CTW / 2; ++ps) {
#pragma unroll
          for (int cta = 0; cta < 2; ++cta)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              uint2 o;
              o.x = enc16x2<F16>(acc2[2 * ps + cta][q * 4 + 0], acc2[2 * ps + cta][q * 4 + 1]);
              o.y = enc16x2<F16>(acc2[2 * ps + cta][q * 4 + 2], acc2[2 * ps + cta][q * 4 + 3]);
              *(uint2*)(stage + c32 * 128 + (((cta * 4 + q) ^ (c32 & 7)) * 16) + 8 * g) = o;
            }
          __builtin_amdgcn_wave_barrier();
          u32x4 rowv[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) rowv[i] = *(const u32x4*)(stage + (rl + 8 * i) * 128 + ((pc ^ rl) * 16));
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (rlive[i]) *(u32x4*)(rptr[i] + ps * 64) = rowv[i];
        }
      }
    }
    __syncthreads();   // the pairs' records and the staging slices are rewritten by the next group
  }
}

// Ordered combine: thread = (token, 8 columns); the token's result rows are contiguous, experts ascending.
template <bool F16 = false>
__global__ __launch_bounds__(256) void combine_kernel(const bf16_t* __restrict__ y, const int32_t* __restrict__ tok_off,
                                                      const int32_t* __restrict__ flag, const bf16_t* __restrict__ x,
                                                      const bf16_t* __restrict__ last_bias, bf16_t* __restrict__ out, int64_t N,
                                                      int D, int add_residual, int singles_done) {
  if (flag[0] == 0) return;
  const int ppr = D / 8;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n = idx / ppr;
  if (n >= N) return;
  const int col = (int)(idx - n * ppr) * 8;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  const int q0 = tok_off[n], q1 = tok_off[n + 1];
  if (singles_done && q1 - q0 == 1) return;   // finished by the experts kernel
  // rows are added in ascending order; eight of them are requested at a time (a token of a small batch may have a
  // couple of hundred, and one load per trip would make the sum a chain of memory round trips)
  int q = q0;
  for (; q + 8 <= q1; q += 8) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *(const uint4*)(y + (int64_t)(q + u) * D + col);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t wd[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += (i & 1) ? dec16_hi<F16>(wd[i >> 1]) : dec16<F16>(wd[i >> 1] & 0xffffu);
    }
  }
  for (; q < q1; ++q) {
    const uint4 v = *(const uint4*)(y + (int64_t)q * D + col);
    const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += (i & 1) ? dec16_hi<F16>(wd[i >> 1]) : dec16<F16>(wd[i >> 1] & 0xffffu);
  }
  if (last_bias != nullptr) {
    const uint4 v = *(const uint4*)(last_bias + col);
    const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += (i & 1) ? dec16_hi<F16>(wd[i >> 1]) : dec16<F16>(wd[i >> 1] & 0xffffu);
  }
  if (add_residual) {
    const uint4 v = *(const uint4*)(x + n * D + col);
    const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += (i & 1) ? dec16_hi<F16>(wd[i >> 1]) : dec16<F16>(wd[i >> 1] & 0xffffu);
  }
  uint4 o;
  o.x = enc16x2<F16>(acc[0], acc[1]); o.y = enc16x2<F16>(acc[2], acc[3]);
  o.z = enc16x2<F16>(acc[4], acc[5]); o.w = enc16x2<F16>(acc[6], acc[7]);
  *(uint4*)(out + n * D + col) = o;
}

// ---------------------------------------------------------------------------------------------------
// Gated experts, expert-major (Gemma shape: D = 2048, experts of at most 64 neurons, no biases):
//   y[pair, :] = routing . (act(x Wg[e]) * (x Wu[e])) Wd[e]      for the 32 pairs of a tile of expert e
// The layer is bound by the weight stream (786 KB per expert against 128 KB of x rows per tile), so the work is dealt to
// keep four independent streams going.  First products: wave w owns ONE 32-neuron tile over all of K -- waves 0,1 the
// gate tiles, waves 2,3 the up tiles -- with x rows read from their gathered positions (the four waves share them
// through the L1) and two register buffers of 8 K steps; nothing is summed across waves.  The up waves hand their tile
// to the gate waves through LDS, which apply the activation, the product and the routing weight and leave H as B
// fragments in LDS.  Second product: wave w owns 512 output columns, 4 column tiles at a time, fragments of the next
// four in flight while the current are multiplied; rows leave through a wave-private LDS tile as whole 256-byte
// segments.  Every pair's row goes to y, tokens with one expert included; the combine kernel sums them.
// ---------------------------------------------------------------------------------------------------
template <int D, int ACT, bool F16 = false>
__global__ __launch_bounds__(256, 2) void experts_gated_sparse_kernel(const SparseArgs A) {
  constexpr int KS1 = D / 16;
  constexpr int NT = 2;          // 32-neuron tiles per projection (expert size <= 64)
  constexpr int CTW = D / 128;   // column tiles per wave
  constexpr int U = 8;           // K steps per register buffer
  static_assert(KS1 % (2 * U) == 0 && CTW % 8 == 0, "buffers alternate in pairs");
  __shared__ int32_t s_tile_off[1025];
  __shared__ int32_t s_offsets[1025];
  __shared__ float upx[2][16][64];
  __shared__ __attribute__((aligned(16))) bf16x8 hs[2 * NT][64];
  __shared__ __attribute__((aligned(16))) u32x4 stage_all[4][32 * 16];
  if (A.flag[0] == 0) return;
  const int E = A.E;
  for (int i = threadIdx.x; i <= E; i += 256) {
    s_tile_off[i] = A.tile_off[i];
    s_offsets[i] = A.offsets[i];
  }
  __syncthreads();
  const int n_tiles = s_tile_off[E];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = lane >> 5, c32 = lane & 31;
  const int xcd = blockIdx.x & 7, wg = blockIdx.x >> 3, nwg = gridDim.x >> 3;   // the grid is a multiple of 8
  const int t_lo = (int)((int64_t)n_tiles * xcd / 8), t_hi = (int)((int64_t)n_tiles * (xcd + 1) / 8);
  for (int T = t_lo + wg; T < t_hi; T += nwg) {
    int lo = 0, hi = E;   // largest e with tile_off[e] <= T
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_tile_off[mid] <= T) lo = mid; else hi = mid;
    }
    const int e = lo;
    const int base = s_offsets[e];
    const int cnt = s_offsets[e + 1] - base;
    const int j0 = (T - s_tile_off[e]) * SP_BT;
    const int rows = (cnt - j0 < SP_BT) ? (cnt - j0) : SP_BT;
    const int pj = base + j0 + (c32 < rows ? c32 : rows - 1);
    const int tok = A.token_idx[pj];
    const int dst = A.pair_dst[pj];
    const float rw = dec16<F16>(A.routing[(int64_t)tok * E + e]);

    // ---- first products: this wave's tile over all of K
    const bf16x8* wf = ((w >> 1) ? A.wus : A.w1s) + ((int64_t)e * KS1 * NT + (w & 1)) * 64 + lane;   // + NT * 64 per K step
    const bf16x8* xrow = (const bf16x8*)(A.x + (int64_t)tok * D) + g;                               // + 2 per K step
    f32x16 acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc1[r] = 0.f;
    bf16x8 xA[U], wA[U], xB[U], wB[U];
    auto fill = [&](bf16x8 (&xb)[U], bf16x8 (&wb)[U], int ks0) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        xb[u] = xrow[2 * (ks0 + u)];
        wb[u] = wf[(int64_t)(ks0 + u) * NT * 64];
      }
    };
    auto multiply = [&](bf16x8 (&xb)[U], bf16x8 (&wb)[U]) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < U; ++u) acc1 = mfma_32x32x16<F16>(wb[u], xb[u], acc1);
    };
    fill(xA, wA, 0);
    for (int ks0 = 0; ks0 < KS1; ks0 += 2 * U) {
      fill(xB, wB, ks0 + U);
      multiply(xA, wA);
      fill(xA, wA, (ks0 + 2 * U < KS1) ? (ks0 + 2 * U) : ks0);   // the last trip re-reads its own steps: in bounds, unused
      multiply(xB, wB);
    }
    // the first column tiles of the second product are requested before the exchange
    const bf16x8* w2f = A.w2s + ((int64_t)e * (D / 32) + w * CTW) * (2 * NT) * 64 + lane;   // [col tile][K step 2 NT][lane]
    bf16x8 fA[4][2 * NT], fB[4][2 * NT];
    auto fill2 = [&](bf16x8 (&f)[4][2 * NT], int ct0) __attribute__((always_inline)) {
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int k = 0; k < 2 * NT; ++k) f[ct][k] = w2f[((ct0 + ct) * (2 * NT) + k) * 64];
    };
    fill2(fA, 0);
    if (w >= 2) {
#pragma unroll
      for (int r = 0; r < 16; ++r) upx[w - 2][r][lane] = acc1[r];
    }
    __syncthreads();
    if (w < 2) {
      float hv[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float gv = (ACT >= 0) ? act_fn<ACT>(acc1[r]) : apply_act(A.act_rt, acc1[r]);
        hv[r] = gv * upx[w][r][lane] * rw;
      }
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint4 pk;
        pk.x = enc16x2<F16>(hv[half * 8 + 0], hv[half * 8 + 1]);
        pk.y = enc16x2<F16>(hv[half * 8 + 2], hv[half * 8 + 3]);
        pk.z = enc16x2<F16>(hv[half * 8 + 4], hv[half * 8 + 5]);
        pk.w = enc16x2<F16>(hv[half * 8 + 6], hv[half * 8 + 7]);
        ((uint4*)hs)[(w * 2 + half) * 64 + lane] = pk;
      }
    }
    __syncthreads();
    bf16x8 hb[2 * NT];
#pragma unroll
    for (int k = 0; k < 2 * NT; ++k) hb[k] = hs[k][lane];

    // ---- second product (transposed): OUT^T[512 columns of this wave, 32 pairs], 4 column tiles per pass
    u32x4* stage = stage_all[w];                    // 32 rows x 256 bytes
    const int rl = lane >> 4, pc = lane & 15;
    bf16_t* rptr[8];
    bool rlive[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int R = rl + 4 * i;
      const int rd = __shfl(dst, R, kWave);
      rptr[i] = A.y + (int64_t)rd * D + w * (D / 4) + pc * 8;
      rlive[i] = R < rows;
    }
    auto pass = [&](bf16x8 (&f)[4][2 * NT], int ct0) __attribute__((always_inline)) {
      f32x16 acc2[4];
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[ct][r] = 0.f;
#pragma unroll
        for (int k = 0; k < 2 * NT; ++k) acc2[ct] = mfma_32x32x16<F16>(f[ct][k], hb[k], acc2[ct]);
      }
      // lane = pair c32, accumulator r = column 8*(r/4) + 4g + r%4 of the tile -> 16-byte piece ct*4 + r/4, half g
      uint2* srow = (uint2*)(stage + c32 * 16);
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint2 o;
          o.x = enc16x2<F16>(acc2[ct][q * 4 + 0], acc2[ct][q * 4 + 1]);
          o.y = enc16x2<F16>(acc2[ct][q * 4 + 2], acc2[ct][q * 4 + 3]);
          srow[(((ct * 4 + q) ^ (c32 & 15)) << 1) + g] = o;
        }
      __builtin_amdgcn_wave_barrier();
      u32x4 rowv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int R = rl + 4 * i;
        rowv[i] = stage[R * 16 + (pc ^ (R & 15))];
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (rlive[i]) *(u32x4*)(rptr[i] + ct0 * 32) = rowv[i];
    };
    for (int ct0 = 0; ct0 < CTW; ct0 += 8) {
      fill2(fB, ct0 + 4);
      pass(fA, ct0);
      fill2(fA, (ct0 + 8 < CTW) ? (ct0 + 8) : ct0);   // the last trip re-reads its own tiles: in bounds, unused
      pass(fB, ct0 + 4);
    }
  }
}

template <bool F16>
static void launch_gated_sparse_experts(const SparseArgs& A, int act, unsigned grid, hipStream_t s) {
  switch (act) {
    case D2DMOE_ACT_GELU_TANH:
      hipLaunchKernelGGL((experts_gated_sparse_kernel<2048, D2DMOE_ACT_GELU_TANH, F16>), dim3(grid), dim3(256), 0, s, A); break;
    case D2DMOE_ACT_RELU:
      hipLaunchKernelGGL((experts_gated_sparse_kernel<2048, D2DMOE_ACT_RELU, F16>), dim3(grid), dim3(256), 0, s, A); break;
    default:
      hipLaunchKernelGGL((experts_gated_sparse_kernel<2048, -1, F16>), dim3(grid), dim3(256), 0, s, A); break;
  }
}

template <int D, int NT, bool F16, bool RT_ACT = false>   // RT_ACT: only the variant with the activation chosen at run time
static hipError_t launch_group_experts(const SparseArgs& A, int act, hipStream_t s) {
  const size_t lds = sg_lds_bytes<NT>(D);
  const unsigned grid = (unsigned)(device_cu_count() * sg_wgs_per_cu(D, NT));
#define D2DMOE_GROUP_LAUNCH(ACTV)                                                                                \
  {                                                                                                              \
    auto kern = experts_mfma_group_kernel<D, NT, ACTV, F16>;                                                     \
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
    if (e != hipSuccess) return e;                                                                               \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, s, A);                                                  \
  }
  if constexpr (RT_ACT) {
    D2DMOE_GROUP_LAUNCH(-1)
  } else {
    switch (act) {
      case D2DMOE_ACT_RELU: D2DMOE_GROUP_LAUNCH(D2DMOE_ACT_RELU) break;
      case D2DMOE_ACT_GELU: D2DMOE_GROUP_LAUNCH(D2DMOE_ACT_GELU) break;
      default: D2DMOE_GROUP_LAUNCH(-1) break;
    }
  }
#undef D2DMOE_GROUP_LAUNCH
  return hipSuccess;
}

void launch_plan_count_scan(const void* routing, int64_t N, int E, int32_t* seg_counts, int32_t* seg_pairs,
                            int32_t* seg_offsets, int32_t* totals, hipStream_t s, bool counts_ready) {
  const int64_t n_seg = cdiv64(N, SP_SEG);
  const unsigned seg_blocks = (unsigned)cdiv64(n_seg, 4);
  const int vpt = (E + 63) / 64;
#define D2DMOE_PLAN_DISPATCH(V)                                                                                          \
  hipLaunchKernelGGL(plan_count_kernel<V>, dim3(seg_blocks), dim3(256), 0, s, (const bf16_t*)routing, seg_counts, seg_pairs, N, \
                     E, n_seg)
  if (counts_ready) {}   // the router kernel has left them there
  else if (vpt <= 1) D2DMOE_PLAN_DISPATCH(1); else if (vpt <= 2) D2DMOE_PLAN_DISPATCH(2); else if (vpt <= 4) D2DMOE_PLAN_DISPATCH(4);
  else if (vpt <= 8) D2DMOE_PLAN_DISPATCH(8); else D2DMOE_PLAN_DISPATCH(16);
#undef D2DMOE_PLAN_DISPATCH
  launch_perm_scan(seg_counts, seg_offsets, totals, E, n_seg, s);
}

void mfma_sparse_plan_counts(const d2dmoe_shape& sh, void* workspace, int32_t** seg_counts, int32_t** seg_pairs) {
  const SparseWorkspace W = sparse_workspace(sh, mfma_sparse_capacity_k(sh));
  *seg_counts = (int32_t*)((char*)workspace + W.seg_counts);
  *seg_pairs = (int32_t*)((char*)workspace + W.seg_pairs);
}

hipError_t launch_mfma_sparse(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                              const void* last_bias, void* out, void* workspace, int max_mean_k, const int** flag_out,
                              hipStream_t s, bool counts_ready) {
  const int cap_k = mfma_sparse_capacity_k(sh);
  if (max_mean_k > cap_k) max_mean_k = cap_k;
  const SparseWorkspace W = sparse_workspace(sh, cap_k);   // sized for the maximum; the flag uses max_mean_k
  const PackedLayout L = packed_layout(sh);
  char* ws = (char*)workspace;
  const char* pk = (const char*)packed;
  const int64_t N = sh.n_tokens;
  const int E = sh.n_experts;
  int32_t* seg_counts = (int32_t*)(ws + W.seg_counts);
  int32_t* seg_offsets = (int32_t*)(ws + W.seg_offsets);
  int32_t* totals = (int32_t*)(ws + W.totals);
  int32_t* seg_pairs = (int32_t*)(ws + W.seg_pairs);
  int32_t* offsets = (int32_t*)(ws + W.offsets);
  int32_t* tile_off = (int32_t*)(ws + W.tile_off);
  int32_t* flag = (int32_t*)(ws + W.flag);
  int32_t* tok_off = (int32_t*)(ws + W.tok_off);
  int32_t* token_idx = (int32_t*)(ws + W.token_idx);
  int32_t* pair_dst = (int32_t*)(ws + W.pair_dst);
  bf16_t* y = (bf16_t*)(ws + W.y);
  const unsigned seg_blocks = (unsigned)cdiv64(W.n_seg, 4);
  // up to 16 384 tokens the scatter gives each segment a workgroup (four waves on its tokens); beyond, the extra
  // workgroups' repeated prologues cost more than the shorter token loops save (measured: -5 us at 4096 tokens, +3.6 us
  // at 50 432)
  const bool split_seg = W.n_seg <= 512;
  const int vpt = (E + 63) / 64;
  launch_plan_count_scan(routing, N, E, seg_counts, seg_pairs, seg_offsets, totals, s, counts_ready);
#define D2DMOE_PLAN_DISPATCH(V)                                                                                          \
  hipLaunchKernelGGL(plan_scatter_kernel<V>, dim3(split_seg ? (unsigned)W.n_seg : seg_blocks), dim3(256), 0, s,          \
                     (const bf16_t*)routing, seg_offsets,                                                                \
                     totals, seg_pairs, offsets, tile_off, flag, tok_off, token_idx, pair_dst, N, E, W.n_seg,           \
                     (max_mean_k == cap_k) ? W.cap : N * (int64_t)max_mean_k, split_seg ? 1 : 0)
  if (vpt <= 1) D2DMOE_PLAN_DISPATCH(1); else if (vpt <= 2) D2DMOE_PLAN_DISPATCH(2); else if (vpt <= 4) D2DMOE_PLAN_DISPATCH(4);
  else if (vpt <= 8) D2DMOE_PLAN_DISPATCH(8); else D2DMOE_PLAN_DISPATCH(16);
#undef D2DMOE_PLAN_DISPATCH
  SparseArgs A;
  A.x = (const bf16_t*)x; A.routing = (const bf16_t*)routing; A.w1s = (const bf16x8*)(pk + L.s1_off);
  A.w2s = (const bf16x8*)(pk + L.s2_off); A.b1s = (const bf16_t*)(pk + L.sb_off); A.offsets = offsets;
  A.tile_off = tile_off; A.token_idx = token_idx; A.pair_dst = pair_dst; A.flag = flag; A.y = y; A.E = E;
  A.act_rt = sh.activation;
  A.tok_off = tok_off; A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out; A.add_residual = sh.add_residual;
  A.wus = (const bf16x8*)(pk + L.su_off);
  const unsigned grid = (unsigned)(8 * device_cu_count());
  const bool f16 = sh.dtype == D2DMOE_F16;
  if (sh.gated) { if (f16) launch_gated_sparse_experts<true>(A, sh.activation, grid, s); else launch_gated_sparse_experts<false>(A, sh.activation, grid, s); }
  else {
    // D = 768 with the activation as a template argument; the wider models (D = 1024: GPT-2 medium, BERT-large, ViT-L;
    // D = 1280: GPT-2 large) with the activation chosen at run time
    hipError_t ge = hipErrorInvalidValue;
#define D2DMOE_GROUP(DD, NTT, RT) (f16 ? launch_group_experts<DD, NTT, true, RT>(A, sh.activation, s) : launch_group_experts<DD, NTT, false, RT>(A, sh.activation, s))
    if (sh.d_model == 1024) ge = (L.nt == 1) ? D2DMOE_GROUP(1024, 1, true) : D2DMOE_GROUP(1024, 2, true);
    else if (sh.d_model == 1280) ge = D2DMOE_GROUP(1280, 1, true);
    else if (L.nt == 1) ge = D2DMOE_GROUP(768, 1, false);
    else if (L.nt == 2) ge = D2DMOE_GROUP(768, 2, false);
    else ge = D2DMOE_GROUP(768, 4, false);
#undef D2DMOE_GROUP
    if (ge != hipSuccess) return ge;
  }
  const int64_t n_threads = N * (sh.d_model / 8);
  if (f16)
    hipLaunchKernelGGL(combine_kernel<true>, dim3((unsigned)cdiv64(n_threads, 256)), dim3(256), 0, s, y, tok_off, flag, (const bf16_t*)x,
                       (const bf16_t*)last_bias, (bf16_t*)out, N, sh.d_model, sh.add_residual, sh.gated ? 0 : 1);
  else
    hipLaunchKernelGGL(combine_kernel<false>, dim3((unsigned)cdiv64(n_threads, 256)), dim3(256), 0, s, y, tok_off, flag, (const bf16_t*)x,
                       (const bf16_t*)last_bias, (bf16_t*)out, N, sh.d_model, sh.add_residual, sh.gated ? 0 : 1);
  *flag_out = flag;
  return hipGetLastError();
}

}  // namespace d2dmoe

