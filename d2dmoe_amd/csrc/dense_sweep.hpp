// The fused experts kernel ("masked dense sweep") as a header: the tile routine, its two kernels and their launcher are
// templates over the model width, instantiated for D = 768 in kernels_mfma.hip and for D = 1024 in
// kernels_dense_wide.hip (two translation units so that they compile side by side).
#pragma once

#include "mfma_common.hpp"

// Build-time forms of the sweep (for comparison runs; the defaults are the product):
//   D2DMOE_SWEEP_DYN  1: a tile works through the blocks of hidden neurons its tokens use (gathered chunks)
//                     0: through every chunk of the packed stream that holds a used expert (fixed chunks)
//   D2DMOE_SWEEP_NW   4: one wave per SIMD; 8: two (D = 768, fixed chunks only)
#ifndef D2DMOE_SWEEP_DYN
#define D2DMOE_SWEEP_DYN 1
#endif
#ifndef D2DMOE_SWEEP_NW
#define D2DMOE_SWEEP_NW 4
#endif

namespace d2dmoe {

// ---------------------------------------------------------------------------------------------------
// Fused experts kernel, token-tile-major ("masked dense sweep").
// Workgroup = 4 waves (one per SIMD), a tile of 64 tokens (or 32: "half tile", used for the last partial round of
// tiles so the machine does not idle through a mostly empty round).  LDS: the x tile as B fragments (96 KB at
// D = 768, resident), one chunk of h as A fragments (32 KB), the routing tile, bias / expert-index tables.
// At D = 1024 the x tile takes 128 KB: the chunk is 128 neurons (h: 16 KB) and the routing tile stays in global memory,
// a chunk's values being requested into registers while the chunk before it is multiplied.
// Per chunk of 256 (128) neurons:
//   GEMM1  wave w: H^T[64 (32) neurons of w, tokens] over K = D      A = W1 fragments (stream), B = x (LDS)
//   epilogue      + b1, activation, x routing[token, expert(neuron)], round to bf16, store as A fragments to LDS
//   GEMM2  wave w: OUT[tokens, D/4 columns of w] += H . W2            A = h (LDS), B = W2 fragments (stream)
// OUT stays in registers across all chunks (ascending neuron = ascending expert order, float32) and is rounded
// once in the final epilogue (+ last_bias, + x).  A tile leaves out what none of its tokens routes to: by blocks of
// 32 neurons gathered into chunks of its own (the default, described at dense_tile below), or by whole chunks of the
// packed stream (uniform branch).
//
// Each wave runs at one wave per SIMD, so memory latency is hidden by software: the weight stream is read MD_RING
// fragments ahead into a register ring (compile-time indices), across phase and chunk boundaries;
// __builtin_amdgcn_sched_barrier pins every refill where it is written.  The two workgroup barriers per chunk wait
// on LDS traffic only, so the global loads in flight survive them; GEMM2 of one chunk and GEMM1 of the next run
// back to back between barriers.
// ---------------------------------------------------------------------------------------------------
struct DenseArgs {
  const bf16_t* x; const bf16_t* routing; const bf16x8* wp; const bf16_t* b1p; const uint8_t* eidx;
  const bf16_t* last_bias; bf16_t* out;
  const int* skip_flag;   // optional device flag: non-zero = the expert-major path handles this call
  float* partial;         // [csplit][part_rows][D] float32 sums of the chunk-split tiles (tokens from part_base on)
  int csplit; int chunks_per_split; int64_t part_base; int64_t part_rows;
  int64_t N; int E; int expert_dim; int n_chunks; int hidden; int act_rt; int add_residual; int n_full; int n_tiles;
  int pf_lines;           // 128-byte lines of the whole weight stream, for the warming reads
};

// What depends on the model width: the chunk of hidden neurons a workgroup multiplies between two barriers, and
// whether the tile's routing rows fit in LDS next to the x tile.
template <int D> struct SweepCfg {
  static constexpr int HC = sweep_chunk(D);       // hidden neurons per chunk
  static constexpr int LOG_HC = (HC == 256) ? 8 : 7;
  static constexpr int RT = HC / 128;             // 32-neuron row tiles of GEMM1 per wave
  static constexpr int KS2 = HC / 16;             // K = 16 steps of GEMM2 per chunk
  static constexpr bool RLDS = (D <= 768);        // routing tile staged in LDS
  // The output tile's accumulators fill the 256 accumulation registers at D = 1024; GEMM1's sums must then live in
  // ordinary vector registers, which the compiler does not arrange by itself (it spills accumulator tiles instead):
  // GEMM1's MFMAs are written as assembly statements with vector-register operands there.
  static constexpr bool VACC = (D > 768);
};

// A wave's stream of 16-byte-per-lane fragments, indexed in units of 16 bytes and read with buffer loads: the stream's
// base sits in a resource descriptor (scalar registers), the position in the stream is a scalar byte offset, and the
// lane's 16 bytes are ONE vector register that never changes -- the walk through the stream costs no vector
// arithmetic and no vector registers for addresses (with plain pointers each group of four fragments takes a 64-bit
// vector add and a register pair; measured at D = 768: 1.6 % of the kernel).
struct StreamPtr {
  __amdgpu_buffer_rsrc_t rsrc; uint32_t loff; int soff;   // soff: bytes, the same in all lanes
  __device__ __forceinline__ bf16x8 operator[](int i) const {
    // (the whole position goes into the scalar offset: one scalar add per load, and the vector offset stays one register)
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)loff, soff + i * 16, 0);
    return __builtin_bit_cast(bf16x8, v);
  }
  __device__ __forceinline__ StreamPtr operator+(int64_t n) const { return {rsrc, loff, soff + (int)n * 16}; }
};

// One MFMA with its accumulator in ordinary vector registers (first: C = 0).  The compiler does not know these are matrix
// instructions: whoever reads the sums with another kind of instruction waits with mfma_vacc_settle() first.
template <bool F16, bool FIRST> __device__ __forceinline__ void mfma_32x32x16_vacc(const bf16x8& a, const bf16x8& b, f32x16& c) {
  if constexpr (FIRST) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  } else {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
}
// The matrix pipe writes its results some cycles after the instruction issues and the hardware does not hold back a
// vector instruction that reads them early (11 wait states for this 8-pass instruction; 18 are spent).  One wait
// serves every tile: volatile statements keep their order, so a reader of any tile comes after the first statement.
__device__ __forceinline__ void mfma_vacc_settle(f32x16& last) { asm volatile("s_nop 15\n\ts_nop 1" : "+v"(last)); }
__device__ __forceinline__ void mfma_vacc_settled(f32x16& other) { asm volatile("" : "+v"(other)); }

// SPLIT: the workgroup handles only chunks [c_begin, c_end) of its tile and leaves its float32 sums, without bias or
// residual, in A.partial[split]; a finishing kernel adds the splits in ascending order.
// NW: waves per workgroup.  4 = one per SIMD, each with a quarter of the chunk's neurons (GEMM1) and of the output columns
// (GEMM2).  8 = two per SIMD, each with an eighth: wave w works on half sub = w % 2 of what wave w / 2 of the 4-wave form
// does and reads the same packed stream (every second W1 fragment, three of every six W2 fragments).
// DYN: the chunks the tile works through are gathered, not the fixed ones of the packed stream.  The unit is a block of
// 32 hidden neurons (a wave's GEMM1 row tile, two K steps of GEMM2).  At staging the tile finds the blocks that hold a
// neuron of any expert some token of the tile routes to, and lists them -- active ones first, ascending, then the
// rest.  "Chunk" v is then blocks list[v * BPC .. v * BPC + BPC) (BPC = blocks per chunk), and the tile stops after the
// last chunk that holds an active block (the inactive blocks that fill it up multiply hidden activations that are all
// zero).  Everything else -- ring, barriers, LDS layout, summation order over ascending neurons -- is as in the fixed
// form, whose chunks are the case list = 0, 1, 2, ...: for a routing that uses every block the two forms run the same
// instructions on the same addresses, and for any routing they give the same bits (the blocks left out would have
// added zeros).  The time of a tile follows the number of distinct experts its 64 tokens use.
template <int D, int ACT, bool ED8, int TT, bool SPLIT = false, bool F16 = false, int NW = 4, bool DYN = false>
__device__ __forceinline__ void dense_tile(const DenseArgs& A, const int64_t tok0, unsigned char* smem_raw,
                                           const int c_begin = 0, const int c_end = 1 << 30, const int split = 0) {
  static_assert(!DYN || NW == 4, "gathered chunks: the four-wave form only");
  constexpr int WS = NW / 4;           // waves that share one packed stream
  constexpr int NT = 64 * NW;          // threads
  constexpr int KS1 = D / 16;          // K steps of GEMM1
  constexpr int CT = D / 128 / WS;     // 32-wide column tiles per wave in GEMM2
  constexpr int HC = SweepCfg<D>::HC, LOG_HC = SweepCfg<D>::LOG_HC, RT = SweepCfg<D>::RT / WS, KS2 = SweepCfg<D>::KS2;
  constexpr bool RLDS = SweepCfg<D>::RLDS, VACC = SweepCfg<D>::VACC;
  static_assert(NW == 4 || (NW == 8 && !VACC && SweepCfg<D>::RT == 2 && (D / 128) % 2 == 0), "8 waves: the D = 768 form only");
  const int E = A.E, n_chunks = A.n_chunks;
  const int64_t N = A.N;
  bf16x8* xs = (bf16x8*)smem_raw;                              // [2][KS1][64]
  bf16x8* hs = xs + 2 * KS1 * 64;                              // [2][KS2][64]
  const int RS = E + 8;                                        // padded row stride (16-byte aligned rows)
  const int HP = n_chunks * HC;
  bf16_t* rs = (bf16_t*)(hs + 2 * KS2 * 64);                   // [64][E+8] routing tile (RLDS)
  bf16_t* b1s = rs + (RLDS ? MD_BM * RS : 0);                  // [HP] first-layer bias
  uint8_t* eis = (uint8_t*)(b1s + HP);                         // [HP] expert index of each neuron
  uint32_t* ebits = (uint32_t*)(eis + HP);                     // [E rounded up to 8] chunks each expert's neurons lie in
  uint32_t* cmask_lds = ebits + ((E + 7) & ~7);                // chunks some token of the tile needs (bit per chunk)
  // DYN: experts some token routes to (bit per expert, in the first 8 words of ebits, which it does not use otherwise),
  // the waves' ballots of active blocks, and the list of blocks
  uint32_t* emask = ebits;
  constexpr int BPC = HC / 32;                                 // blocks per chunk
  constexpr int MAXB = MD_MAX_CHUNKS * 8;                      // most blocks a layer can have (256: block numbers are bytes)

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int w = __builtin_amdgcn_readfirstlane(t >> 6);   // wave index, known to the compiler to be the same in all lanes
  const int g = lane >> 5, c32 = lane & 31;
  uint8_t* blist = (uint8_t*)(cmask_lds + 2) + w * MAXB;  // DYN: this wave's own copy of the block list
  constexpr int NW1 = RT * KS1;        // W1 fragments per (wave, chunk)
  constexpr int NW2 = KS2 * CT;        // W2 fragments per (wave, chunk)
  constexpr int PIECES = WS * (NW1 + NW2);   // fragments per chunk of a packed stream
  constexpr int R = MD_RING / WS;      // fragments in flight per wave (the same bytes per CU in both forms)
  constexpr int BM = 32 * TT;
  static_assert(NW1 % R == 0 && NW2 % R == 0, "every phase must start at ring slot 0");
  // position in a chunk of the packed stream of this wave's s-th W1 / W2 fragment, less what depends on sub
  auto P1 = [](int s) constexpr { return (s / RT) * (RT * WS) + s % RT; };
  auto P2 = [](int s) constexpr { return (s / CT) * (CT * WS) + s % CT; };

  // ---- staging.  Every global load of the tile's inputs is issued up front, in the order the data is needed:
  // routing pieces and the two tables (short, and the active-chunk mask hangs on them), the x tile, then the weight
  // stream of the first chunk (almost every tile starts at chunk 0; if its first active chunk turns out to be another
  // one the ring is reloaded below).  Loads complete in order, so each stage below waits only for what precedes it.
  //
  // A wave stages RW consecutive rows of the tile.  Lane (r = lane & 7, c = lane >> 3) takes row r of a block of 8
  // rows and the 16-byte pieces c, c + 8, c + 16 ... of it: 8 lanes read 128 contiguous bytes of a row, 8 lanes write
  // 128 contiguous bytes of LDS (the rows of a fragment), and all further addresses are compile-time offsets from a
  // handful of lane values -- this part of the kernel is bound by instruction issue, not by memory.
  // Rows past the end of the batch are read from the last row instead (rows never mix, and their results are not
  // stored).
  typedef StreamPtr Stream;
  // this wave's stream: a raw buffer of 32-bit words covering the wave's part of the packed weights
  const int wb = w / WS, sub = w % WS;
  const Stream wbase{__builtin_amdgcn_make_buffer_rsrc((void*)(A.wp + (int64_t)wb * n_chunks * PIECES * 64), 0,
                                                       n_chunks * PIECES * 1024, 0x00020000), (uint32_t)lane * 16u, 0};
  // a chunk's W1 fragments of this wave start at chunkA(c), its W2 fragments at chunkA(c) + W2OFF (units of 16 bytes)
  auto chunkA = [&](int c) __attribute__((always_inline)) { return wbase + ((int64_t)c * PIECES + sub * RT) * 64; };
  const int W2OFF = (WS * NW1 + sub * CT - sub * RT) * 64;
  // Where a chunk's fragments are.  Fixed chunks: `a` (above).  Gathered chunks (DYN): per block, in units of 16 bytes
  // from the start of ALL waves' streams -- oA[rt]: the W1 fragments of this wave's row tile rt (K step ks at
  // + ks * RT * 64), oB[p]: this wave's W2 fragments of the chunk's p-th block (half h, column tile ct at
  // + (h * CT + ct) * 64); blk[rt]: the block itself (for the bias / expert-index tables).
  struct ChunkSrc { Stream a; int oA[RT]; int oB[DYN ? BPC : 1]; int blk[RT]; uint32_t lo, hi; };
  const Stream wall{__builtin_amdgcn_make_buffer_rsrc((void*)A.wp, 0, MD_WAVES * n_chunks * PIECES * 1024, 0x00020000),
                    (uint32_t)lane * 16u, 0};
  // lo / hi: the chunk's block numbers, one byte each (BPC = 4: lo only)
  auto src_of_blocks = [&](uint32_t lo, uint32_t hi) __attribute__((always_inline)) {
    ChunkSrc c;
    c.a = wbase; c.lo = lo; c.hi = hi;
#pragma unroll
    for (int p = 0; p < BPC; ++p) {
      const int b = (int)(((p < 4 ? lo : hi) >> ((p & 3) * 8)) & 0xffu);
      c.oB[DYN ? p : 0] = ((w * n_chunks + b / BPC) * PIECES + NW1 + 2 * (b % BPC) * CT) * 64;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int pos = w * RT + rt;
      const int b = (int)(((pos < 4 ? lo : hi) >> ((pos & 3) * 8)) & 0xffu);
      const int q = b % BPC;
      c.blk[rt] = b;
      c.oA[rt] = (((q / RT) * n_chunks + b / BPC) * PIECES + q % RT) * 64;
    }
    return c;
  };
  auto blocks_of_fixed = [&](int c, uint32_t& lo, uint32_t& hi) __attribute__((always_inline)) {   // chunk c as it is packed
    lo = (uint32_t)(c * BPC) * 0x01010101u + 0x03020100u;
    hi = (uint32_t)(c * BPC) * 0x01010101u + 0x07060504u;
  };
  auto blocks_of_listed = [&](int v, uint32_t& lo, uint32_t& hi) __attribute__((always_inline)) {  // chunk v of the list
    const uint32_t* bl = (const uint32_t*)blist + v * (BPC / 4);
    lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)bl[0]);
    hi = (BPC > 4) ? (uint32_t)__builtin_amdgcn_readfirstlane((int)bl[BPC > 4 ? 1 : 0]) : 0u;
  };
  // the s-th W1 / W2 fragment of a chunk (s: position in this wave's sequence)
  auto w1_frag = [&](const ChunkSrc& c, int s) __attribute__((always_inline)) {
    if constexpr (DYN) return wall[c.oA[s % RT] + (s / RT) * (RT * 64)];
    else return c.a[P1(s) * 64];
  };
  auto w2_frag = [&](const ChunkSrc& c, int s) __attribute__((always_inline)) {
    if constexpr (DYN) return wall[c.oB[(s / CT) / 2] + (((s / CT) % 2) * CT + s % CT) * 64];
    else return c.a[W2OFF + P2(s) * 64];
  };
  bf16x8 ring[R];
  const int first_guess = SPLIT ? c_begin : 0;
  const int last_row = (int)((N - 1 - tok0) < (int64_t)(BM - 1) ? (N - 1 - tok0) : (int64_t)(BM - 1));
  {
    constexpr int RW = BM / NW;                     // rows per wave
    constexpr int RR = RW < 8 ? RW : 8;             // rows per block (8; 4 where a wave has only 4 rows)
    constexpr int RB = RW / RR;                     // row blocks per wave
    constexpr int LPR = 64 / RR;                    // lanes per row
    constexpr int XK = D / 8 / LPR;                 // 16-byte pieces of a row per lane (12 with 8 lanes per row)
    constexpr int RK = 32 / LPR;                    // routing pieces of a row per lane (E <= 256)
    constexpr int TB1 = MD_MAX_CHUNKS * 32 / NT, TEI = MD_MAX_CHUNKS * 16 / NT;   // table pieces per thread
    const int r8 = lane % RR, c8l = lane / RR;
    const bool wide = (E & 7) == 0;                 // routing rows are whole 16-byte pieces
    const int EP = E >> 3;
    if (t == 0) *cmask_lds = 0u;
    if constexpr (DYN) {
      if (t < 8) emask[t] = 0u;
    } else {
      for (int e = t; e < E; e += NT) {
        const int h0 = e * A.expert_dim;
        ebits[e] = (1u << (h0 >> LOG_HC)) | (1u << ((h0 + A.expert_dim - 1) >> LOG_HC));
      }
    }
    int mrow[RB];                                   // tile row of each row block, clamped to the last real row
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = w * RW + rb * RR + r8;
      mrow[rb] = m < last_row ? m : last_row;
    }
    u32x4 rv[RB][RK];
    if (wide) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const u32x4* rrow = (const u32x4*)(A.routing + (tok0 + mrow[rb]) * E);
#pragma unroll
        for (int kb = 0; kb < RK; ++kb)
          if (kb * LPR < EP) rv[rb][kb] = rrow[c8l + kb * LPR < EP ? c8l + kb * LPR : 0];   // lanes past the row: piece 0
      }
    }
    u32x4 tb[TB1], te[TEI];
#pragma unroll
    for (int k = 0; k < TB1; ++k) {
      const int i = t + k * NT;
      tb[k] = ((const u32x4*)A.b1p)[i < HP / 8 ? i : 0];
    }
#pragma unroll
    for (int k = 0; k < TEI; ++k) {
      const int i = t + k * NT;
      te[k] = ((const u32x4*)A.eidx)[i < HP / 16 ? i : 0];
    }
    // Warming reads of the weight stream: workgroup b touches lines 2 NT b .. 2 NT b + 2 NT - 1 (one 4-byte load per
    // 128-byte line, two per thread; past the end: line 0).  All workgroups of a round walk the stream in step, a ring of
    // MD_RING fragments ahead of the MFMAs -- enough for lines that wait in an L2 or in the memory-side cache, not for
    // lines that come from memory, which is where a layer's weights are when other layers' work has gone through the
    // caches since its last call.  The first round's workgroups between them touch the whole stream while they stage
    // their tiles; by the time the stream gets there, the lines are on the near side of memory.
    uint32_t pf[2];
    {
      const uint32_t* wl = (const uint32_t*)A.wp;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int l = ((int)blockIdx.x * 2 + k) * NT + t;
        pf[k] = wl[(int64_t)(l < A.pf_lines ? l : 0) * 32];
      }
    }
    u32x4 xv[RB][XK];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const u32x4* xrow = (const u32x4*)(A.x + (tok0 + mrow[rb]) * D) + c8l;
#pragma unroll
      for (int kb = 0; kb < XK; ++kb) xv[rb][kb] = xrow[kb * LPR];
    }
    lds_barrier();   // chunk bits per expert written, mask cleared
    __builtin_amdgcn_sched_barrier(0);
    uint32_t need = 0u;                             // chunks the rows staged by this thread need
    uint32_t ebyte[RK];                             // DYN: which of the 8 experts of each of its pieces they route to
#pragma unroll
    for (int kb = 0; kb < RK; ++kb) ebyte[kb] = 0u;
    if (wide) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int m = w * RW + rb * RR + r8;
#pragma unroll
        for (int kb = 0; kb < RK; ++kb) {
          if (kb * LPR < EP && c8l + kb * LPR < EP) {
            const int piece = c8l + kb * LPR;
            const u32x4 r4 = rv[rb][kb];
            if constexpr (RLDS) *(u32x4*)(rs + m * RS + piece * 8) = r4;
            const uint32_t wd[4] = {r4.x, r4.y, r4.z, r4.w};
            if constexpr (DYN) {
#pragma unroll
              for (int i = 0; i < 8; ++i)
                ebyte[kb] |= (wd[i >> 1] & ((i & 1) ? 0x7fff0000u : 0x7fffu)) != 0 ? (1u << i) : 0u;
            } else {
              const u32x4 eb0 = *(const u32x4*)(ebits + piece * 8);
              const u32x4 eb1 = *(const u32x4*)(ebits + piece * 8 + 4);
              const uint32_t eb[8] = {eb0.x, eb0.y, eb0.z, eb0.w, eb1.x, eb1.y, eb1.z, eb1.w};
#pragma unroll
              for (int i = 0; i < 8; ++i)
                need |= (wd[i >> 1] & ((i & 1) ? 0x7fff0000u : 0x7fffu)) != 0 ? eb[i] : 0u;
            }
          }
        }
      }
      if constexpr (DYN) {
#pragma unroll
        for (int kb = 0; kb < RK; ++kb) {
          const int piece = c8l + kb * LPR;
          if (ebyte[kb] != 0u)
            __hip_atomic_fetch_or((__attribute__((address_space(3))) uint32_t*)(emask + (piece >> 2)),
                                  ebyte[kb] << ((piece & 3) * 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < TB1; ++k) {
      const int i = t + k * NT;
      if (i < HP / 8) ((u32x4*)b1s)[i] = tb[k];
    }
#pragma unroll
    for (int k = 0; k < TEI; ++k) {
      const int i = t + k * NT;
      if (i < HP / 16) ((u32x4*)eis)[i] = te[k];
    }
    __builtin_amdgcn_sched_barrier(0);
    {
      ChunkSrc first;
      if constexpr (DYN) {
        uint32_t lo, hi;
        blocks_of_fixed(first_guess, lo, hi);
        first = src_of_blocks(lo, hi);
      } else {
        first.a = chunkA(first_guess);
      }
#pragma unroll
      for (int i = 0; i < R; ++i) ring[i] = w1_frag(first, i);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!wide) {
      for (int i = t; i < BM * E; i += NT) {
        const int m = i / E, e = i - m * E;
        const bf16_t r1 = A.routing[(tok0 + (m < last_row ? m : last_row)) * E + e];
        if constexpr (RLDS) rs[m * RS + e] = r1;
        if constexpr (DYN) {
          if ((r1 & 0x7fff) != 0)
            __hip_atomic_fetch_or((__attribute__((address_space(3))) uint32_t*)(emask + (e >> 5)), 1u << (e & 31),
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
          if ((r1 & 0x7fff) != 0) need |= ebits[e];
        }
      }
    }
    if (!DYN && need != 0u)
      __hip_atomic_fetch_or((__attribute__((address_space(3))) uint32_t*)cmask_lds, need, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_WORKGROUP);
    // x fragments: piece kk of row m goes to fragment kk / 2 (K step), slot (m & 31) + 32 * (kk & 1)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = w * RW + rb * RR + r8;
      u32x4* xdst = (u32x4*)xs + ((m >> 5) * KS1 + (c8l >> 1)) * 64 + (m & 31) + 32 * (c8l & 1);
#pragma unroll
      for (int kb = 0; kb < XK; ++kb) xdst[kb * (LPR / 2) * 64] = xv[rb][kb];
    }
    asm volatile("" :: "v"(pf[0]), "v"(pf[1]));      // the warming reads' registers are theirs until they have landed
  }
  lds_barrier();
  // Active chunks as a bit mask, the same in every wave: the chunk loop walks its set bits.
  // (DYN: a mask of the chunks of the list that hold an active block -- the first ceil(active blocks / BPC))
  uint32_t cmask;
  if constexpr (DYN) {
    // Block b is active iff one of the experts with a neuron in it is routed to by some token of the tile.  Every wave
    // works the list out for itself (lane l looks at blocks l, l + 64, ...) and keeps its own copy in LDS: no exchange
    // between the waves, no further barrier.
    const int n_blocks = n_chunks * BPC;
    const int Ed = A.expert_dim;
    unsigned long long bal[MAXB / 64];
    bool on[MAXB / 64];
    int total = 0;
#pragma unroll
    for (int k = 0; k < MAXB / 64; ++k) {
      const int b = lane + 64 * k;
      on[k] = false;
      bal[k] = 0ull;
      if (64 * k < n_blocks) {                       // uniform
        if (b < n_blocks) {
          const int e_lo = (32 * b) / Ed;
          int e_hi = (32 * b + 31) / Ed;
          e_hi = e_hi < E - 1 ? e_hi : E - 1;
          for (int e = e_lo; e <= e_hi; ++e) on[k] |= ((emask[e >> 5] >> (e & 31)) & 1u) != 0;
        }
        bal[k] = __ballot(on[k]);
        total += __popcll(bal[k]);
      }
    }
    int before = 0;                                  // active blocks in the passes before this one
#pragma unroll
    for (int k = 0; k < MAXB / 64; ++k) {
      const int b = lane + 64 * k;
      if (64 * k < n_blocks) {
        const int below = before + __popcll(bal[k] & ((1ull << lane) - 1ull));
        if (b < n_blocks) blist[on[k] ? below : total + (b - below)] = (uint8_t)b;
        before += __popcll(bal[k]);
      }
    }
    const int n_vc = (total + BPC - 1) / BPC;
    cmask = (n_vc >= 32) ? ~0u : ((1u << n_vc) - 1u);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the list is read back below by the wave that wrote it
  } else {
    cmask = __builtin_amdgcn_readfirstlane(*cmask_lds);
  }
  if constexpr (SPLIT) {
    const uint32_t below_end = (c_end >= 32) ? ~0u : ((1u << c_end) - 1u);
    cmask &= below_end & ~((1u << c_begin) - 1u);
  }
  const int n_act = __popc(cmask);

  f32x16 acc2[TT][CT];
#pragma unroll
  for (int a = 0; a < TT; ++a)
#pragma unroll
    for (int b = 0; b < CT; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[a][b][r] = 0.f;

  if (n_act > 0) {
    f32x16 acc1[RT][TT];  // GEMM1 accumulators [row-tile][token tile]
    const int first_chunk = __builtin_ctz(cmask);
    auto src_of_chunk = [&](int c) __attribute__((always_inline)) {
      if constexpr (DYN) {
        uint32_t lo, hi;
        blocks_of_listed(c, lo, hi);
        return src_of_blocks(lo, hi);
      } else {
        ChunkSrc r;
        r.a = chunkA(c);
        return r;
      }
    };
    ChunkSrc cur = src_of_chunk(first_chunk);
    bool guessed = first_chunk == first_guess;
    if constexpr (DYN) {
      uint32_t glo, ghi;
      blocks_of_fixed(first_guess, glo, ghi);
      guessed = cur.lo == glo && (BPC <= 4 || cur.hi == ghi);
    }
    if (!guessed) {
#pragma unroll
      for (int i = 0; i < R; ++i) ring[i] = w1_frag(cur, i);
    }

    // Without the routing tile in LDS: the routing values a lane's accumulators are multiplied by (its tokens, the experts
    // of its rows), raw 16-bit patterns, requested one chunk ahead.
    constexpr int NRQ = ED8 ? 4 : 16;
    uint32_t rpre[TT][RT][NRQ];
    auto routing_request = [&](const ChunkSrc& src_r, int chunk_r, int g, int c32) __attribute__((always_inline)) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        const int m = tt * 32 + c32;
        const char* rtile = (const char*)(A.routing + tok0 * E);   // the same in all lanes; byte offsets from it below
        const uint32_t rrow = (uint32_t)((m < last_row ? m : last_row) * E) * 2u;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int hb = (DYN ? src_r.blk[rt] * 32 : chunk_r * HC + w * (32 * RT) + rt * 32) + 4 * g + 8 * q;
            if (ED8) {
              rpre[tt][rt][q] = *(const bf16_t*)(rtile + (rrow + 2u * eis[hb & ~7]));
            } else {
              const uint32_t e4 = *(const uint32_t*)(eis + hb);
#pragma unroll
              for (int i = 0; i < 4; ++i) rpre[tt][rt][q * 4 + i] = *(const bf16_t*)(rtile + (rrow + 2u * ((e4 >> (8 * i)) & 0xff)));
            }
          }
        }
      }
    };

    // This lane's 16 bytes of the first x / h fragment of each token tile.  Where the tiles span more than the 64 KB an
    // LDS instruction's immediate offset reaches, the compiler would keep one address per fragment in registers (and
    // spill them): the tile offsets are made opaque there, so that every fragment is one base register + an immediate.
    // (x tile 0 starts at the lane's own offset, both h tiles lie within one immediate's reach of the first)
    const bf16x8* xrow[TT];
    const bf16x8* hrow[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      uint32_t xo = (uint32_t)(tt * KS1 * 64 + lane), ho = (uint32_t)lane;
      if constexpr (VACC) {
        if (tt > 0) asm volatile("" : "+v"(xo));
        if (tt == 0) asm volatile("" : "+v"(ho));
      } else {
        ho += (uint32_t)(tt * KS2 * 64);
      }
      xrow[tt] = xs + xo;
      hrow[tt] = (VACC && tt > 0) ? hrow[0] + tt * KS2 * 64 : hs + ho;
    }

    for (int ci = 0; ci < n_act; ++ci) {
      const int chunk = __builtin_ctz(cmask);
      cmask &= cmask - 1;
      const ChunkSrc nxt = (cmask != 0) ? src_of_chunk(__builtin_ctz(cmask)) : cur;
      // Where registers are short (VACC), what the epilogue derives from the lane index -- table and h-tile addresses,
      // routing rows -- is recomputed from a fresh copy of it in every chunk instead of being kept across the products.
      int lane_c = lane;
      if constexpr (VACC) asm volatile("" : "+v"(lane_c));
      const int g = lane_c >> 5, c32 = lane_c & 31;
      // first neuron of this lane's accumulator rows in row tile rt
      auto hb_of = [&](const ChunkSrc& c, int chunk_c, int rt) __attribute__((always_inline)) {
        if constexpr (DYN) return c.blk[rt] * 32 + 4 * g;
        else return chunk_c * HC + w * (32 * RT) + rt * 32 + 4 * g;
      };

      // epilogue state, filled and consumed in slices between MFMAs
      uint2 e_bias[4];     // 4 bf16 biases per accumulator quad
      uint32_t e_idx[4];   // expert index: one per quad (ED8) or four packed uint8
      float e_rq[TT][ED8 ? 4 : 16];
      float e_hv[TT][16];
      auto epi_load_tables = [&](int rt) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int hb = hb_of(cur, chunk, rt) + 8 * q;
          e_bias[q] = *(const uint2*)(b1s + hb);
          // Ed multiple of 8: the aligned block of 8 neurons a quad pair covers belongs to one expert, the same for
          // every lane, so one routing value per (quad, token tile) serves four accumulator rows
          e_idx[q] = ED8 ? (uint32_t)eis[hb & ~7] : *(const uint32_t*)(eis + hb);
        }
      };
      auto epi_load_routing = [&](int rt) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          if constexpr (RLDS) {
            const bf16_t* rrow = rs + (tt * 32 + c32) * RS;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              if (ED8) {
                e_rq[tt][q] = dec16<F16>(rrow[e_idx[q]]);
              } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) e_rq[tt][q * 4 + i] = dec16<F16>(rrow[(e_idx[q] >> (8 * i)) & 0xff]);
              }
            }
          } else {
#pragma unroll
            for (int i = 0; i < NRQ; ++i) e_rq[tt][i] = dec16<F16>(rpre[tt][rt][i]);
          }
        }
      };
      auto epi_math = [&](int rt, int q) __attribute__((always_inline)) {
        const float b0 = dec16<F16>(e_bias[q].x & 0xffffu), b1 = dec16_hi<F16>(e_bias[q].x);
        const float b2 = dec16<F16>(e_bias[q].y & 0xffffu), b3 = dec16_hi<F16>(e_bias[q].y);
        const float bias[4] = {b0, b1, b2, b3};
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int r = q * 4 + i;
            float v = acc1[rt][tt][r] + bias[i];
            v = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(A.act_rt, v);
            e_hv[tt][r] = v * (ED8 ? e_rq[tt][q] : e_rq[tt][r]);
          }
        }
      };
      auto epi_store = [&](int rt) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            uint4 pk;
            pk.x = enc16x2<F16>(e_hv[tt][half * 8 + 0], e_hv[tt][half * 8 + 1]);
            pk.y = enc16x2<F16>(e_hv[tt][half * 8 + 2], e_hv[tt][half * 8 + 3]);
            pk.z = enc16x2<F16>(e_hv[tt][half * 8 + 4], e_hv[tt][half * 8 + 5]);
            pk.w = enc16x2<F16>(e_hv[tt][half * 8 + 6], e_hv[tt][half * 8 + 7]);
            const int ks2 = (w * RT + rt) * 2 + half;
            ((uint4*)hs)[(tt * KS2 + ks2) * 64 + lane_c] = pk;
          }
        }
      };
      // GEMM1 of the chunk whose stream starts at `pre` (its W1 fragments; the refills run on into its W2 fragments)
      auto gemm1 = [&](const ChunkSrc& pre) __attribute__((always_inline)) {
        if constexpr (!VACC) {
#pragma unroll
          for (int a = 0; a < RT; ++a)
#pragma unroll
            for (int b = 0; b < TT; ++b)
#pragma unroll
              for (int r = 0; r < 16; ++r) acc1[a][b][r] = 0.f;
        }
        bf16x8 xb[TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) xb[tt] = xrow[tt][0];
        static_for<0, KS1>([&](auto ks_c) __attribute__((always_inline)) {
          constexpr int ks = decltype(ks_c)::value;
          bf16x8 a[RT];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) a[rt] = ring[(RT * ks + rt) % R];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {   // the refills run on into the chunk's own W2 fragments
            constexpr int s = RT * ks, sr = s + R;
            ring[(s + rt) % R] = (sr + rt < NW1) ? w1_frag(pre, sr + rt) : w2_frag(pre, sr + rt - NW1);
          }
          constexpr int kn = (ks + 1 < KS1) ? ks + 1 : ks;      // x fragments of the next step, read one step ahead
          bf16x8 nxb[TT];
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) nxb[tt] = xrow[tt][kn * 64];
#pragma unroll
          for (int tt = 0; tt < TT; ++tt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
              if constexpr (VACC) mfma_32x32x16_vacc<F16, ks == 0>(a[rt], xb[tt], acc1[rt][tt]);
              else acc1[rt][tt] = mfma_32x32x16<F16>(a[rt], xb[tt], acc1[rt][tt]);
            }
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) xb[tt] = nxb[tt];
          __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (VACC) {
          mfma_vacc_settle(acc1[RT - 1][TT - 1]);
#pragma unroll
          for (int a = 0; a < RT; ++a)
#pragma unroll
            for (int b = 0; b < TT; ++b)
              if (a != RT - 1 || b != TT - 1) mfma_vacc_settled(acc1[a][b]);
        }
      };
      // GEMM2 of the current chunk; refills run on into the next chunk's W1 fragments
      auto gemm2 = [&]() __attribute__((always_inline)) {
        bf16x8 ha[TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) ha[tt] = hrow[tt][0];
        static_for<0, KS2>([&](auto j_c) __attribute__((always_inline)) {
          constexpr int j = decltype(j_c)::value;
          constexpr int jn = (j + 1 < KS2) ? j + 1 : j;         // h fragments of the next step, read one step ahead
          bf16x8 nha[TT];
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) nha[tt] = hrow[tt][jn * 64];
          static_for<0, CT>([&](auto ct_c) __attribute__((always_inline)) {
            constexpr int ct = decltype(ct_c)::value;
            constexpr int s = j * CT + ct;      // position in this phase; refill position s + R
            const bf16x8 b = ring[s % R];
            ring[s % R] = (s + R < NW2) ? w2_frag(cur, s + R) : w1_frag(nxt, s + R - NW2);
#pragma unroll
            for (int tt = 0; tt < TT; ++tt)
              acc2[tt][ct] = mfma_32x32x16<F16>(ha[tt], b, acc2[tt][ct]);
          });
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) ha[tt] = nha[tt];
          __builtin_amdgcn_sched_barrier(0);
        });
      };

      if (ci == 0) {
        if constexpr (!RLDS) routing_request(cur, chunk, g, c32);
        gemm1(cur);
      }
      lds_barrier();   // every wave has finished reading the previous h tile
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        epi_load_tables(rt);
        epi_load_routing(rt);
#pragma unroll
        for (int q = 0; q < 4; ++q) epi_math(rt, q);
        epi_store(rt);
      }
      lds_barrier();   // h tile complete
      // (the values of the last chunk are requested once more instead of branching round the loads)
      if constexpr (!RLDS) routing_request(nxt, cmask != 0 ? __builtin_ctz(cmask) : chunk, g, c32);
      gemm2();
      if (ci + 1 < n_act) gemm1(nxt);
      cur = nxt;
    }
  }

  // ---- final epilogue: the accumulators are rounded to bf16 once, AFTER + last_bias (+ x) in float32, and leave as
  // whole rows.  One pass per 32-token tile: every wave writes its D/NW columns of the pass's rows to LDS as float
  // [32][D + 4] (bias added on the way: a lane's accumulators share CT columns), then wave w takes rows 8w .. 8w + 7
  // (4w .. 4w + 3 with 8 waves) with the lane mapping of the staging above -- lane (r, c) reads 8 consecutive columns
  // c, c + 8, ... of row r, adds the residual, rounds, stores 16 bytes; 8 lanes cover 128 contiguous bytes of an output
  // row.  The residual rows are requested before the pass's LDS traffic; the read loop has no branches and no address
  // arithmetic.
  {
    constexpr int OS = D + 4;                       // row stride in floats (+16 bytes: rows shift by 4 banks, so the
    float* ot = (float*)smem_raw;                   // 8 rows a wave reads at once cover all 32); fits in x + h regions
    static_assert((size_t)32 * OS * 4 <= (size_t)(2 * KS1 * 64 + 2 * KS2 * 64) * 16, "out staging fits");
    constexpr int FR = 32 / NW;                     // rows of a pass per wave
    constexpr int FL = 64 / FR;                     // lanes per row
    constexpr int OP = D / 8 / FL;                  // 8-column pieces per thread and pass
    const int r8 = lane % FR, c8l = lane / FR;
    const bool with_bias = !SPLIT && A.last_bias != nullptr;
    const bool with_res = !SPLIT && A.add_residual != 0;
    float lb[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
      lb[ct] = with_bias ? dec16<F16>(A.last_bias[w * (D / NW) + ct * 32 + c32]) : 0.f;
    const int row = w * FR + r8;                    // row of the pass this thread finishes
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const int64_t n = tok0 + tt * 32 + row;
      const bool live = n < N;
      u32x4 xr[OP];
      if (with_res) {
        const u32x4* xrow = (const u32x4*)(A.x + (live ? n : N - 1) * D) + c8l;
#pragma unroll
        for (int k = 0; k < OP; ++k) xr[k] = xrow[k * FL];
      }
      lds_barrier();                                // previous readers of this LDS region are done
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const int col = w * (D / NW) + ct * 32 + c32;
#pragma unroll
        for (int r = 0; r < 16; ++r)
          ot[(8 * (r / 4) + 4 * g + (r % 4)) * OS + col] = with_bias ? acc2[tt][ct][r] + lb[ct] : acc2[tt][ct][r];
      }
      lds_barrier();
      const float* orow = ot + row * OS + c8l * 8;
      u32x4 o[OP];
      float4 pv0[OP], pv1[OP];
#pragma unroll
      for (int k = 0; k < OP; ++k) {
        pv0[k] = *(const float4*)(orow + k * FL * 8);
        pv1[k] = *(const float4*)(orow + k * FL * 8 + 4);
        if constexpr (!SPLIT) {
          float v[8] = {pv0[k].x, pv0[k].y, pv0[k].z, pv0[k].w, pv1[k].x, pv1[k].y, pv1[k].z, pv1[k].w};
          if (with_res) {
            const uint32_t xw[4] = {xr[k].x, xr[k].y, xr[k].z, xr[k].w};
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] += (i & 1) ? dec16_hi<F16>(xw[i >> 1]) : dec16<F16>(xw[i >> 1] & 0xffffu);
          }
          o[k].x = enc16x2<F16>(v[0], v[1]); o[k].y = enc16x2<F16>(v[2], v[3]);
          o[k].z = enc16x2<F16>(v[4], v[5]); o[k].w = enc16x2<F16>(v[6], v[7]);
        }
      }
      if (live) {
        if constexpr (SPLIT) {
          float* prow = A.partial + ((int64_t)split * A.part_rows + (n - A.part_base)) * D + c8l * 8;
#pragma unroll
          for (int k = 0; k < OP; ++k) {
            *(float4*)(prow + k * FL * 8) = pv0[k];
            *(float4*)(prow + k * FL * 8 + 4) = pv1[k];
          }
        } else {
          u32x4* grow = (u32x4*)(A.out + n * D) + c8l;
#pragma unroll
          for (int k = 0; k < OP; ++k) grow[k * FL] = o[k];
        }
      }
    }
  }
}

// Values that are the same in every lane but reach a device function in vector registers (its arguments do): moved to
// scalar registers, so that what is derived from them -- buffer resources, loop bounds, branch conditions -- is scalar
// again.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform(int64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}
template <typename T> __device__ __forceinline__ T* uniform(T* p) { return (T*)(uintptr_t)uniform((int64_t)(uintptr_t)p); }

// Out-of-line copy of the tile routine for the variant below (keeps its register allocation apart from the loop).
template <int D, int ACT, bool ED8, int TT, bool F16>
__device__ __attribute__((noinline)) void dense_tile_call(const DenseArgs& A, const int64_t tok0, unsigned char* smem_raw) {
  constexpr bool DYN = D2DMOE_SWEEP_DYN != 0;
  DenseArgs U;
  U.x = uniform(A.x); U.routing = uniform(A.routing); U.wp = uniform(A.wp); U.b1p = uniform(A.b1p); U.eidx = uniform(A.eidx);
  U.last_bias = uniform(A.last_bias); U.out = uniform(A.out); U.skip_flag = nullptr; U.partial = nullptr;
  U.csplit = 1; U.chunks_per_split = 0; U.part_base = 0; U.part_rows = 0;
  U.N = uniform(A.N); U.E = uniform(A.E); U.expert_dim = uniform(A.expert_dim); U.n_chunks = uniform(A.n_chunks);
  U.hidden = uniform(A.hidden); U.act_rt = uniform(A.act_rt); U.add_residual = uniform(A.add_residual);
  U.pf_lines = uniform(A.pf_lines);
  U.n_full = 0; U.n_tiles = 0;
  dense_tile<D, ACT, ED8, TT, false, F16, 4, DYN>(U, uniform(tok0), smem_raw);
}

// The same sweep launched as one workgroup per CU that walks the tiles in launch order.  Used where the launch is
// usually a no-op (the fall-back behind the expert-major path): a skipped call then retires after one round of empty
// workgroups instead of one per tile.
template <int D, int ACT, bool ED8, bool F16 = false>
__global__ __launch_bounds__(256, 1) void experts_mfma_dense_walk_kernel(const DenseArgs A) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  if (A.skip_flag != nullptr && *A.skip_flag != 0) return;   // uniform over the whole grid
  for (int b = blockIdx.x; b < A.n_tiles; b += gridDim.x) {
    if (b < A.n_full)
      dense_tile_call<D, ACT, ED8, 2, F16>(A, (int64_t)b * 64, smem_raw);
    else
      dense_tile_call<D, ACT, ED8, 1, F16>(A, (int64_t)A.n_full * 64 + (int64_t)(b - A.n_full) * 32, smem_raw);
    __syncthreads();   // the next tile's staging overwrites the LDS the final epilogue just read
  }
}

// Workgroups [0, n_full) take tiles of 64 tokens.  The tokens left over after the last full round of the machine go to
// tiles of 32; if those would still leave most CUs idle, each of them is dealt to csplit workgroups by chunk ranges,
// which leave float32 sums in A.partial for the finishing kernel.
template <int D, int ACT, bool ED8, bool F16 = false, int NW = 4, bool DYN = false>
__global__ __launch_bounds__(64 * NW, 1) void experts_mfma_dense_kernel(const DenseArgs A) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  if (A.skip_flag != nullptr && *A.skip_flag != 0) return;   // uniform over the whole grid
  const int b = blockIdx.x;
  if (b < A.n_full) {
    dense_tile<D, ACT, ED8, 2, false, F16, NW, DYN>(A, (int64_t)b * 64, smem_raw);
  } else if (A.csplit <= 1) {
    dense_tile<D, ACT, ED8, 1, false, F16, NW, DYN>(A, (int64_t)A.n_full * 64 + (int64_t)(b - A.n_full) * 32, smem_raw);
  } else {
    const int idx = b - A.n_full;
    const int tile = idx / A.csplit, split = idx % A.csplit;
    const int c_begin = split * A.chunks_per_split;
    dense_tile<D, ACT, ED8, 1, true, F16, NW, DYN>(A, (int64_t)A.n_full * 64 + (int64_t)tile * 32, smem_raw, c_begin,
                                              c_begin + A.chunks_per_split, split);
  }
}

struct DenseTiling {
  int64_t n_full, n_half;   // tiles of 64 and of 32 tokens
  int csplit, per;          // workgroups per tile of 32 and chunks per workgroup (1, n_chunks: not split)
  int64_t part_base, part_rows;   // tokens covered by split tiles
};
DenseTiling dense_tiling(const d2dmoe_shape& sh, bool allow_split);
size_t dense_lds_bytes(const d2dmoe_shape& sh);

template <int D, int ACT, bool ED8, bool F16>
static inline hipError_t launch_dense_cfg(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                   const void* last_bias, void* out, const int* skip_flag, void* workspace,
                                   size_t workspace_bytes, hipStream_t s) {
  const PackedLayout L = packed_layout(sh);
  const char* base = (const char*)packed;
  const size_t lds = dense_lds_bytes(sh);
  if (lds > 160 * 1024) return hipErrorInvalidValue;
  const int cus = device_cu_count();
  // Behind the expert-major path the launch is usually a no-op: one workgroup per CU walks the tiles, so a skipped call
  // retires after one round of empty workgroups.  With big experts (the reference's benchmark shape, swept over
  // densities) the fall-back runs as often as not, and the walk costs 15 % per tile: the ordinary grid there.
  const bool walk = skip_flag != nullptr && sh.expert_dim <= 64;
  const bool allow_split = !walk && workspace != nullptr && workspace_bytes >= mfma_dense_workspace_bytes(sh);
  const DenseTiling T = dense_tiling(sh, allow_split);
  constexpr int NW = (D == 768) ? D2DMOE_SWEEP_NW : 4;   // waves per workgroup of the ordinary grid
  constexpr bool DYN = D2DMOE_SWEEP_DYN && NW == 4;
  auto kern = walk ? experts_mfma_dense_walk_kernel<D, ACT, ED8, F16> : experts_mfma_dense_kernel<D, ACT, ED8, F16, NW, DYN>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  DenseArgs A;
  A.x = (const bf16_t*)x; A.routing = (const bf16_t*)routing; A.wp = (const bf16x8*)(base + L.w_off);
  A.b1p = (const bf16_t*)(base + L.b1_off); A.eidx = (const uint8_t*)(base + L.eidx_off);
  A.last_bias = (const bf16_t*)last_bias; A.out = (bf16_t*)out; A.N = sh.n_tokens; A.E = sh.n_experts; A.expert_dim = sh.expert_dim;
  A.n_chunks = L.n_chunks; A.hidden = L.hidden; A.act_rt = sh.activation; A.add_residual = sh.add_residual;
  A.n_full = (int)T.n_full; A.n_tiles = (int)(T.n_full + T.n_half); A.skip_flag = skip_flag;
  A.partial = (float*)workspace; A.csplit = T.csplit; A.chunks_per_split = T.per;
  A.part_base = T.part_base; A.part_rows = T.part_rows;
  A.pf_lines = (int)((size_t)MD_WAVES * L.n_chunks * L.pieces * 64 * 16 / 128);
  int64_t grid = T.n_full + T.n_half * T.csplit;
  if (walk && A.n_tiles > cus) grid = cus;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(walk ? 256 : 64 * NW), lds, s, A);
  e = hipGetLastError();
  if (e != hipSuccess || T.csplit <= 1) return e;
  return launch_sum_partials(A.partial, last_bias, (const bf16_t*)x + T.part_base * sh.d_model,
                             (bf16_t*)out + T.part_base * sh.d_model, T.part_rows, sh.d_model, T.csplit, sh.add_residual, s,
                             sh.dtype, skip_flag);
}

template <int D, int ACT>
static inline hipError_t launch_dense_act(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                   const void* last_bias, void* out, const int* skip_flag, void* workspace,
                                   size_t workspace_bytes, hipStream_t s) {
  if (sh.dtype == D2DMOE_F16) {
    if (sh.expert_dim % 8 == 0)
      return launch_dense_cfg<D, ACT, true, true>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
    return launch_dense_cfg<D, ACT, false, true>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
  }
  if (sh.expert_dim % 8 == 0)
    return launch_dense_cfg<D, ACT, true, false>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
  return launch_dense_cfg<D, ACT, false, false>(sh, x, routing, packed, last_bias, out, skip_flag, workspace, workspace_bytes, s);
}

}  // namespace d2dmoe
