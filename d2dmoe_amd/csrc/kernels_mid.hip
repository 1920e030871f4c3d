// Compacted two-kernel bf16 MFMA path for routing of middling density (a few to a few dozen experts per token), where
// a token tile touches every expert but each expert only a fraction of the tile's tokens.  Work follows the routed
// (token, expert) pairs, as in the reference's grouped kernels (moe_impls.py:124-133, 270-293), without gathering an
// x row or writing an output row per pair:
//
//   plan      per segment of 32 tokens the routed-token count per expert, and its prefix over segments (shared with the
//             expert-major path); everything else the kernels derive themselves
//   up        expert-stationary first layer.  A workgroup holds the W1 fragments of 8 experts in registers (one expert
//             per wave) and walks a range of 32-token tiles; a tile of x is copied into LDS once (asynchronously, two
//             buffers) and every wave gathers, for its expert, the tile's routed tokens as the B operand of
//             v_mfma_f32_16x16x32_bf16 -- compaction costs nothing, a lane just reads another row.  Bias, activation and
//             routing weight in registers; the hidden rows (32 bf16 per pair) and the token of every pair go to the
//             pair's place in the expert-major order (expert ascending, tokens ascending inside an expert).
//   down      output-stationary second layer.  A workgroup owns a tile of tokens x 128 output columns as float32 in LDS;
//             for every expert (ascending) it multiplies the tile's compacted hidden rows with that expert's W2 and adds
//             the 16-pair x 16-column results to the rows of their tokens.  A wave owns its columns exclusively, so every
//             output element is summed by one wave in program order: ascending expert order in float32, one rounding
//             after + last_bias (+ x) -- deterministic, the order of the reference's merge kernel (moe_impls.py:499-514).
//
// Fragment layouts of the 16x16x32 bf16 MFMA on a 64-lane wave (q = lane / 16, c = lane % 16):
//   A (16 x 32): lane holds row c,    k = 8q .. 8q+7         B (32 x 16): lane holds column c, k = 8q .. 8q+7
//   C (16 x 16): lane holds column c, rows 4q + r, r = 0..3
#include "mfma_common.hpp"

namespace d2dmoe {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int MID_UP_WAVES = 8;        // experts per workgroup of the first layer
constexpr int MID_TILE = SP_SEG;       // tokens per x tile of the first layer = one plan segment
constexpr int MID_DS = 128;            // output columns per workgroup of the second layer
constexpr int MID_OS = MID_DS + 4;     // row stride of the float32 output tile (rows shift by 4 banks)
constexpr int MID_RING = 4;            // batches of the second layer kept in flight per wave (nine loads each; the
                                       // hardware counts at most 63 outstanding loads per wave)
constexpr int MID_BATCH = 4;           // groups of 16 pairs per batch

bool mfma_mid_supported(const d2dmoe_shape& sh) {
  if (sh.dtype != D2DMOE_BF16 || sh.gated) return false;
  if (sh.d_model != 768) return false;
  // the first layer deals 8 experts to a workgroup; the second lists up to 8 batches per expert in LDS
  return sh.expert_dim <= MID_HROW && sh.n_experts <= 256 && sh.n_experts % MID_UP_WAVES == 0;
}

struct MidWorkspace {
  int64_t n_seg, cap;
  size_t seg_counts, seg_offsets, totals, seg_pairs, offsets, flag, token_idx, hc, total;
};

static MidWorkspace mid_workspace(const d2dmoe_shape& sh) {
  MidWorkspace W;
  const int64_t N = sh.n_tokens;
  const int E = sh.n_experts;
  W.n_seg = cdiv64(N, SP_SEG);
  W.cap = N * (int64_t)(E < MID_MAX_MEAN_K ? E : MID_MAX_MEAN_K);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off += (bytes + 255) / 256 * 256; return o; };
  W.seg_counts = take((size_t)W.n_seg * E * 4);
  W.seg_offsets = take((size_t)W.n_seg * E * 4);
  W.totals = take((size_t)E * 4);
  W.seg_pairs = take((size_t)W.n_seg * 4);
  W.offsets = take((size_t)(E + 1) * 4);
  W.flag = take(16);
  W.token_idx = take((size_t)W.cap * 4);
  W.hc = take((size_t)W.cap * MID_HROW * 2);
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
  const int32_t* seg_offsets; const int32_t* totals; int32_t* offsets; int32_t* flag; int32_t* token_idx; bf16_t* hc;
  const bf16_t* last_bias; bf16_t* out;
  int64_t N; int64_t cap; int E; int n_seg; int tiles_per_chunk; int n_chunks; int n_groups; int act_rt; int add_residual;
  int t2_segs;   // plan segments per token tile of the second layer
};

// Loads whose completion is waited for by hand: the compiler's own bookkeeping gives up on rings of loads carried round
// a loop (it waits for every load in flight, which serialises the kernel on memory latency).  A register written by
// one of these is touched by nothing until wait_loads<N>() has named it.
__device__ __forceinline__ void load16_async(bf16x8& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void load4_async(int& dst, const void* p) {
  asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}

// ---------------------------------------------------------------------------------------------------
// First layer.  512 threads = 8 waves (two per SIMD); wave w holds the W1 fragments of expert 8*group + w in 192
// registers (with more experts per wave the weights spill into the accumulation registers of the matrix unit, and every
// MFMA then pays for copies out of them).  Three tile buffers in LDS (32 tokens x 768 dimensions, 48 KB each)
// are filled by global_load_lds (a wave instruction moves 64 x 16 bytes to 1 KB of consecutive LDS, whatever the lanes'
// global addresses), two tiles ahead of the one being multiplied: a trip multiplies tile t, meets at a barrier, refills
// the buffer it has just left with tile t + 3, waits until its own pieces of tile t + 1 have landed and meets again.
// Rows are not padded; instead the eight 16-byte pieces of every 128 bytes of a row are stored XOR-ed with the row
// number, so that the 16 rows a B fragment reads (same pieces, arbitrary rows) spread over the banks.
// With a tile come its routing values for the workgroup's 8 experts (16 bytes per token) and the 8 experts' positions
// at the start of the tile.
// ---------------------------------------------------------------------------------------------------
constexpr int MID_BUFS = 3;
constexpr int MID_UP_THREADS = 512;
constexpr int MID_EPW = MID_UP_WAVES / (MID_UP_THREADS / 64);   // experts per wave

template <int D, int ACT>
__global__ __launch_bounds__(MID_UP_THREADS) void mid_up_kernel(const MidArgs A) {
  constexpr int NW = MID_UP_THREADS / 64;
  constexpr int KS = D / 32;                              // K steps of 32
  constexpr int ROWB = D * 2;                             // bytes of a row
  constexpr int TILEB = MID_TILE * ROWB;                  // 48 KB
  constexpr int PIECES = ROWB / 16;                       // 16-byte pieces per row
  constexpr int CHUNKS = MID_TILE * PIECES / 64;          // 1 KB chunks per tile
  constexpr int CPW = CHUNKS / NW;                        // chunks per wave
  constexpr int METAB = 1024;                             // per tile: routing [32][8] bf16, then positions [8] int32
  static_assert(CHUNKS % NW == 0 && PIECES % 8 == 0, "tile copy splits evenly over the waves");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* meta = smem + MID_BUFS * TILEB;                        // [MID_BUFS][METAB]
  uint32_t* slot_tab = (uint32_t*)(meta + MID_BUFS * METAB);            // [8 experts][32]: tile row | routing value << 16
  unsigned char* scratch_slot = (unsigned char*)(slot_tab + MID_UP_WAVES * 32);   // [NW][1 KB]: copies nobody reads
  float* bias_lds = (float*)(scratch_slot + NW * 1024);                 // [8 experts][32]
  const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int q = lane >> 4, s16 = lane & 15;
  // workgroups that share a range of tiles sit on one XCD (consecutive block ids go round the XCDs)
  const int xcd = blockIdx.x & 7, jb = blockIdx.x >> 3;
  const int chunk = xcd + 8 * (jb / A.n_groups), group = jb % A.n_groups;
  const int E = A.E;
  const int64_t N = A.N;
  const int e0 = group * MID_UP_WAVES + w * MID_EPW;      // E is a multiple of 8
  // the experts' offsets in the expert-major order and the number of routed pairs, from the per-expert totals
  int before[MID_EPW], all = 0;
#pragma unroll
  for (int x = 0; x < MID_EPW; ++x) before[x] = 0;
  for (int i = lane; i < E; i += 64) {
    const int c = A.totals[i];
    all += c;
#pragma unroll
    for (int x = 0; x < MID_EPW; ++x) before[x] += (i < e0 + x) ? c : 0;
  }
  all = wave_sum_i32(all);
#pragma unroll
  for (int x = 0; x < MID_EPW; ++x) before[x] = wave_sum_i32(before[x]);
  const bool ok = (int64_t)all <= A.cap;
  if (blockIdx.x == 0) {   // published for the second layer and the fall-back
    for (int i = t; i <= E; i += MID_UP_THREADS) {
      int sum = 0;
      for (int k = 0; k < i; ++k) sum += A.totals[k];
      A.offsets[i] = sum;
    }
    if (t == 0) A.flag[0] = ok ? 1 : 0;
  }
  if (!ok || chunk >= A.n_chunks) return;
  const int t_begin = chunk * A.tiles_per_chunk;
  const int t_end = (t_begin + A.tiles_per_chunk < A.n_seg) ? (t_begin + A.tiles_per_chunk) : A.n_seg;
  if (t_begin >= t_end) return;

  // Every wave issues the same CPW + 1 loads per tile (the wait below counts them): CPW pieces of x, and one more that
  // only matters in wave 0 -- the tile's routing values and positions.
  auto issue_tile = [&](int tile_rel) __attribute__((always_inline)) {
    const int tr = t_begin + tile_rel;
    const int tile = tr < t_end ? tr : t_end - 1;         // past the end: the last tile again, into a buffer nobody reads
    const int64_t tb = (int64_t)tile * MID_TILE;
    const int last = (int)((N - 1 - tb) < (int64_t)(MID_TILE - 1) ? (N - 1 - tb) : (int64_t)(MID_TILE - 1));
    unsigned char* buf = smem + (tile_rel % MID_BUFS) * TILEB;
    const bf16_t* tbase = A.x + tb * D;                   // uniform
    static_for<0, CPW>([&](auto i_c) __attribute__((always_inline)) {
      constexpr int i = decltype(i_c)::value;
      // This wave copies rows 4w .. 4w + 3 (six chunks of 64 pieces, 96 pieces to a row): chunk i, lane -> physical
      // piece -> row and piece inside the row, with the divisions by 96 worked out by hand
      static_assert(PIECES == 96 && CPW == 6, "chunk -> row pattern below");
      const bool hi = lane >= 32;
      const int roff = (i % 3 == 0) ? (i / 3) * 2 : (i % 3 == 1) ? ((i / 3) * 2 + (hi ? 1 : 0)) : (i / 3) * 2 + 1;
      const int pcol = (i % 3 == 0) ? lane : (i % 3 == 1) ? (hi ? lane - 32 : lane + 64) : lane + 32;
      const int row = 4 * w + roff;
      const int ccol = (pcol & ~7) | ((pcol ^ row) & 7);
      const int rr = row < last ? row : last;             // rows past the end of the batch: the last row again (unused)
      __builtin_amdgcn_global_load_lds(tbase + (rr * D + ccol * 8), (lds_void*)(buf + (w * CPW + i) * 1024), 16, 0, 0);
      __builtin_amdgcn_sched_barrier(0);   // one address at a time: the weights leave few registers
    });
    {
      // lanes 0..31: 16 bytes of routing row (tb + lane); lanes 32, 33: the 8 experts' positions; the rest repeat lane 0
      const int rr = (lane < 32) ? (lane < last ? lane : last) : 0;
      const unsigned char* g = (const unsigned char*)(A.routing + (tb + rr) * E + group * MID_UP_WAVES);
      if (lane == 32 || lane == 33)
        g = (const unsigned char*)(A.seg_offsets + (int64_t)tile * E + group * MID_UP_WAVES) + (lane - 32) * 16;
      unsigned char* mdst = (w == 0) ? (meta + (tile_rel % MID_BUFS) * METAB) : (scratch_slot + w * 1024);
      __builtin_amdgcn_global_load_lds(g, (lds_void*)mdst, 16, 0, 0);
    }
  };

#pragma unroll
  for (int u = 0; u < MID_BUFS; ++u) issue_tile(u);
  bf16x8 wf[MID_EPW][KS][2];
#pragma unroll
  for (int x = 0; x < MID_EPW; ++x) {
    const bf16x8* wp = A.w1f + (int64_t)(e0 + x) * KS * 2 * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      wf[x][ks][0] = wp[(ks * 2 + 0) * 64];
      wf[x][ks][1] = wp[(ks * 2 + 1) * 64];
    }
  }
  // the 8 experts' biases (32 neurons each, float32) wait in LDS for the epilogues
  if (lane < MID_HROW) {
#pragma unroll
    for (int x = 0; x < MID_EPW; ++x)
      bias_lds[(w * MID_EPW + x) * MID_HROW + lane] = bf16_to_f32(A.b1s[(int64_t)(e0 + x) * MID_HROW + lane]);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  const int n_tiles = t_end - t_begin;
  for (int tr = 0; tr < n_tiles; ++tr) {
    const int tile = t_begin + tr;
    const unsigned char* buf = smem + (tr % MID_BUFS) * TILEB;
    const unsigned char* mt = meta + (tr % MID_BUFS) * METAB;
    const int64_t tok = (int64_t)tile * MID_TILE + (lane & 31);
    int a[MID_EPW];           // routed tokens of the expert in the tile
    int64_t pos0[MID_EPW];
#pragma unroll
    for (int x = 0; x < MID_EPW; ++x) {
      const int ex = w * MID_EPW + x;                      // expert slot inside the workgroup
      const uint32_t rv = (lane < 32 && tok < N) ? (uint32_t)((const bf16_t*)mt)[(lane & 31) * 8 + ex] : 0u;
      const bool on = (rv & 0x7fffu) != 0u;
      const unsigned long long mask = __ballot(on);
      a[x] = __popcll(mask);
      // position among the routed tokens = routed lanes below this one
      const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
      if (on) slot_tab[ex * 32 + rank] = (uint32_t)lane | (rv << 16);
      pos0[x] = (int64_t)before[x] + ((const int32_t*)(mt + 512))[ex];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    static_for<0, MID_EPW>([&](auto x_c) __attribute__((always_inline)) {
      constexpr int x = decltype(x_c)::value;
      for (int g0 = 0; g0 < a[x]; g0 += 16) {              // uniform: groups of 16 routed tokens
        const int idx = g0 + s16;
        const uint32_t ent = slot_tab[(w * MID_EPW + x) * 32 + ((idx < a[x]) ? idx : g0)];
        const int row = (int)(ent & 31u);
        const unsigned char* base = buf + row * ROWB;
        const int o0 = ((q ^ (row & 7)) << 4), o1 = o0 ^ 64;
        f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
        // B fragments are read a few K steps ahead of the MFMAs that use them
        constexpr int AHEAD = 2;
        bf16x8 bq[AHEAD];
#pragma unroll
        for (int ks = 0; ks < AHEAD; ++ks) bq[ks] = *(const bf16x8*)(base + (ks >> 1) * 128 + ((ks & 1) ? o1 : o0));
        static_for<0, KS>([&](auto ks_c) __attribute__((always_inline)) {
          constexpr int ks = decltype(ks_c)::value;
          const bf16x8 b = bq[ks % AHEAD];
          if constexpr (ks + AHEAD < KS)
            bq[ks % AHEAD] = *(const bf16x8*)(base + ((ks + AHEAD) >> 1) * 128 + (((ks + AHEAD) & 1) ? o1 : o0));
          acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[x][ks][0], b, acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[x][ks][1], b, acc1, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        });
        const float rw = __uint_as_float(ent & 0xffff0000u);
        const float* bl = bias_lds + (w * MID_EPW + x) * MID_HROW + 4 * q;
        bf16_t* hrow = A.hc + (pos0[x] + idx) * MID_HROW + 4 * q;
        const bool live = idx < a[x];
        // one row tile after the other (neurons 4q + r, then 16 + 4q + r): bias, activation, routing weight, rounding
        static_for<0, 2>([&](auto rt_c) __attribute__((always_inline)) {
          constexpr int rt = decltype(rt_c)::value;
          const f32x4 bias = *(const f32x4*)(bl + rt * 16);
          float h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float v = (rt == 0 ? acc0[r] : acc1[r]) + bias[r];
            h[r] = ((ACT >= 0) ? act_fn<ACT>(v) : apply_act(A.act_rt, v)) * rw;
          }
          uint2 pk;
          pk.x = pack2_bf16(h[0], h[1]); pk.y = pack2_bf16(h[2], h[3]);
          if (live) *(uint2*)(hrow + rt * 16) = pk;
          __builtin_amdgcn_sched_barrier(0);
        });
        if (live && q == 0) A.token_idx[pos0[x] + idx] = (int32_t)((int64_t)tile * MID_TILE + row);
      }
    });
    // (barriers without a memory fence: a fence would wait for every load in flight, the refills included)
    lds_barrier();            // every wave has left this tile's buffer
    issue_tile(tr + MID_BUFS);
    // this wave's pieces of the NEXT tile have landed once at most the loads of the two tiles issued after it are still
    // in flight; the stores of this trip are older than the refill, so they only make the wait stricter
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"((MID_BUFS - 1) * (CPW + 1)) : "memory");
    lds_barrier();
  }
}

// ---------------------------------------------------------------------------------------------------
// Second layer.  512 threads = 8 waves (two per SIMD); wave w owns columns [16w, 16w + 16) of the workgroup's 128.  The
// tile's routed pairs are cut into batches of up to 64 pairs of one expert, listed in expert order; a wave keeps MID_RING
// batches in flight (hidden fragments, tokens, the expert's W2^T fragment).  Groups of one expert hold different
// tokens, so a batch's read-add-write of the output tile has no overlap inside it; batches follow each other in program
// order, and LDS executes a wave's instructions in order, so a later batch sees an earlier one's sums.
// ---------------------------------------------------------------------------------------------------
struct MidBatch {
  bf16x8 h[MID_BATCH];   // hidden rows of up to MID_BATCH groups of 16 pairs, as B fragments
  int tok[MID_BATCH];    // the pairs' tokens
  bf16x8 aw;             // the expert's W2^T fragment for this wave's column tile
  int n;                 // valid pairs in the batch (0: past the end)
};
constexpr int MID_LOADS = 2 * MID_BATCH + 1;   // loads per batch
constexpr int MID_DOWN_THREADS = 512;

template <int D>
__global__ __launch_bounds__(MID_DOWN_THREADS) void mid_down_kernel(const MidArgs A) {
  constexpr int NS = D / MID_DS;      // column slices
  constexpr int CT = D / 16;          // column tiles of 16
  constexpr int BP = 16 * MID_BATCH;  // pairs per batch
  static_assert(MID_DS / 16 == MID_DOWN_THREADS / 64, "one column tile per wave");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  if (A.flag[0] == 0) return;         // uniform over the grid: the dense sweep runs instead
  const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
  const int q = lane >> 4, s16 = lane & 15;
  const int E = A.E;
  const int64_t N = A.N;
  const int rows = A.t2_segs * SP_SEG;
  const int slice = blockIdx.x % NS;
  const int tile2 = blockIdx.x / NS;
  const int64_t tb = (int64_t)tile2 * rows;
  const int seg0 = tile2 * A.t2_segs, seg1 = seg0 + A.t2_segs;
  float* ot = (float*)smem;                                  // [rows][MID_OS]
  int32_t* s_lo = (int32_t*)(ot + (size_t)rows * MID_OS);    // [E] first pair of the expert inside this tile
  int32_t* s_cnt = s_lo + E;                                 // [E] pairs of the expert inside this tile
  int32_t* s_boff = s_cnt + E;                               // [E + 1] first batch of the expert
  int2* s_desc = (int2*)(s_boff + ((E + 2) & ~1));           // [batches + 2 MID_RING + 2] first pair, pairs | expert << 8
  for (int i = t; i < rows * MID_OS / 4; i += MID_DOWN_THREADS) ((f32x4*)ot)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int e = t; e < E; e += MID_DOWN_THREADS) {
    const int lo = A.offsets[e] + A.seg_offsets[(int64_t)seg0 * E + e];
    const int hi = (seg1 < A.n_seg) ? (A.offsets[e] + A.seg_offsets[(int64_t)seg1 * E + e]) : A.offsets[e + 1];
    s_lo[e] = lo;
    s_cnt[e] = hi - lo;
  }
  __syncthreads();
  // The batch list: the main loop then has nothing data-dependent in its control flow.  One wave scans the batch counts.
  if (w == 0) {
    int run = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int nb = (e < E) ? (s_cnt[e] + BP - 1) / BP : 0;
      int incl = nb;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
      }
      if (e < E) s_boff[e] = run + incl - nb;
      run += __shfl(incl, 63, 64);
    }
    if (lane == 0) s_boff[E] = run;
  }
  __syncthreads();
  const int n_batches = s_boff[E];
  for (int e = t; e < E; e += MID_DOWN_THREADS) {
    const int lo = s_lo[e], cnt = s_cnt[e], b0 = s_boff[e];
    for (int b = 0; b * BP < cnt; ++b) {
      const int n = (cnt - b * BP) < BP ? (cnt - b * BP) : BP;
      s_desc[b0 + b] = make_int2(lo + b * BP, n | (e << 8));
    }
  }
  for (int i = t; i < 2 * MID_RING + 2; i += MID_DOWN_THREADS) s_desc[n_batches + i] = make_int2(0, 0);   // past the end: empty
  __syncthreads();

  const int ct = slice * (MID_DS / 16) + w;
  // Every fetch issues the same MID_LOADS loads whatever the batch holds (addresses clamped to pairs that exist).
  auto fetch = [&](MidBatch& b, int2 ds) __attribute__((always_inline)) {
    const int lo = __builtin_amdgcn_readfirstlane(ds.x);
    const int ne = __builtin_amdgcn_readfirstlane(ds.y);
    b.n = ne & 0xff;
    const int ee = ne >> 8;
    const int last = b.n > 0 ? b.n - 1 : 0;
    load16_async(b.aw, A.w2f + ((int64_t)ee * CT + ct) * 64 + lane);
#pragma unroll
    for (int gg = 0; gg < MID_BATCH; ++gg) {
      const int i = gg * 16 + s16;
      const int64_t slot = lo + (i < last ? i : last);
      load16_async(b.h[gg], A.hc + slot * MID_HROW + q * 8);
      load4_async(b.tok[gg], A.token_idx + slot);
    }
  };
  // names every register of the batch, so that nothing that reads them can be moved ahead of the wait
  auto wait_batch = [&](MidBatch& b) __attribute__((always_inline)) {
    static_assert(MID_BATCH == 4, "operand list below");
    asm volatile("s_waitcnt vmcnt(%9)"
                 : "+v"(b.aw), "+v"(b.h[0]), "+v"(b.h[1]), "+v"(b.h[2]), "+v"(b.h[3]), "+v"(b.tok[0]), "+v"(b.tok[1]),
                   "+v"(b.tok[2]), "+v"(b.tok[3])
                 : "n"((MID_RING - 1) * MID_LOADS)
                 : "memory");
  };

  MidBatch ring[MID_RING];
  static_for<0, MID_RING>([&](auto j_c) __attribute__((always_inline)) {
    fetch(ring[decltype(j_c)::value], s_desc[decltype(j_c)::value]);
  });
  int2 dcur = s_desc[MID_RING];       // the batch the next refill fetches; read one trip ahead of its use
  float* obase = ot + w * 16 + 4 * q;
  for (int i0 = 0; i0 < n_batches; i0 += MID_RING) {
    static_for<0, MID_RING>([&](auto j_c) __attribute__((always_inline)) {
      constexpr int j = decltype(j_c)::value;
      MidBatch& b = ring[j];
      wait_batch(b);
      const int2 dnext = s_desc[i0 + j + MID_RING + 1];   // ahead of the reads below: it is back when they are
      f32x4 y[MID_BATCH], v[MID_BATCH];
      float* addr[MID_BATCH];
#pragma unroll
      for (int gg = 0; gg < MID_BATCH; ++gg) {
        if (gg * 16 < b.n) {          // uniform
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
          y[gg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.aw, b.h[gg], z, 0, 0, 0);
          addr[gg] = obase + (int)(b.tok[gg] - tb) * MID_OS;
          v[gg] = *(const f32x4*)addr[gg];
        }
      }
#pragma unroll
      for (int gg = 0; gg < MID_BATCH; ++gg) {
        if (gg * 16 < b.n) {
          if (gg * 16 + s16 < b.n)     // pairs past the end of the batch hold a copy of its last pair: not added
            *(f32x4*)addr[gg] = v[gg] + y[gg];
        }
      }
      // the refill stays behind the batch's last use and writes the registers it has just left
      __builtin_amdgcn_sched_barrier(0);
      fetch(b, dcur);
      dcur = dnext;
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the refills past the end
  __syncthreads();

  // rows leave as bf16 after + last_bias (+ x): 16 threads per row, 8 columns each
  const int live = (int)((N - tb) < (int64_t)rows ? (N - tb) : (int64_t)rows);
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
static hipError_t launch_mid_up(const MidArgs& A, unsigned grid, size_t lds, hipStream_t s) {
  hipError_t e = hipFuncSetAttribute((const void*)mid_up_kernel<768, ACT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((mid_up_kernel<768, ACT>), dim3(grid), dim3(MID_UP_THREADS), lds, s, A);
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
  A.offsets = (int32_t*)(ws + W.offsets); A.flag = (int32_t*)(ws + W.flag); A.token_idx = (int32_t*)(ws + W.token_idx);
  A.hc = (bf16_t*)(ws + W.hc); A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out;
  A.N = N; A.cap = W.cap; A.E = E; A.n_seg = (int)W.n_seg; A.act_rt = sh.activation; A.add_residual = sh.add_residual;
  launch_plan_count_scan(routing, N, E, (int32_t*)(ws + W.seg_counts), (int32_t*)(ws + W.seg_pairs),
                         (int32_t*)(ws + W.seg_offsets), (int32_t*)(ws + W.totals), s);
  // first layer: groups of 8 experts x ranges of tiles, about one workgroup per CU
  A.n_groups = (E + MID_UP_WAVES - 1) / MID_UP_WAVES;
  int n_chunks = cus / A.n_groups;
  if (n_chunks < 1) n_chunks = 1;
  if (n_chunks > A.n_seg) n_chunks = A.n_seg;
  A.tiles_per_chunk = (A.n_seg + n_chunks - 1) / n_chunks;
  A.n_chunks = (A.n_seg + A.tiles_per_chunk - 1) / A.tiles_per_chunk;
  // second layer: tiles of 256 tokens, or 64 while those would leave CUs without work
  A.t2_segs = (cdiv64(N, 256) * (sh.d_model / MID_DS) >= cus) ? 8 : 2;
  const unsigned grid1 = (unsigned)(8 * A.n_groups * ((A.n_chunks + 7) / 8));
  // three tile buffers, their routing values and positions, the experts' slot tables, the waves' scratch slots, the biases
  const size_t lds1 = (size_t)MID_BUFS * MID_TILE * sh.d_model * 2 + MID_BUFS * 1024 + MID_UP_WAVES * 32 * 4 +
                      (MID_UP_THREADS / 64) * 1024 + MID_UP_WAVES * MID_HROW * 4;
  hipError_t e;
  switch (sh.activation) {
    case D2DMOE_ACT_RELU: e = launch_mid_up<D2DMOE_ACT_RELU>(A, grid1, lds1, s); break;
    case D2DMOE_ACT_GELU: e = launch_mid_up<D2DMOE_ACT_GELU>(A, grid1, lds1, s); break;
    default: e = launch_mid_up<-1>(A, grid1, lds1, s); break;
  }
  if (e != hipSuccess) return e;
  const int rows2 = A.t2_segs * SP_SEG;
  const size_t lds2 = (size_t)rows2 * MID_OS * 4 + (size_t)(3 * E + 4) * 4 +
                      (size_t)(E * (rows2 / (16 * MID_BATCH)) + 2 * MID_RING + 2) * 8;
  e = hipFuncSetAttribute((const void*)mid_down_kernel<768>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2);
  if (e != hipSuccess) return e;
  const unsigned grid2 = (unsigned)(cdiv64(N, rows2) * (sh.d_model / MID_DS));
  hipLaunchKernelGGL((mid_down_kernel<768>), dim3(grid2), dim3(MID_DOWN_THREADS), lds2, s, A);
  *flag_out = A.flag;
  return hipGetLastError();
}

}  // namespace d2dmoe
