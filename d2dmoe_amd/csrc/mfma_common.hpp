// Shared pieces of the bf16 MFMA kernels (gfx950): vector types, tile constants, the packed-weight layout, small
// device helpers.
#pragma once

#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace d2dmoe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));   // 16 raw bytes that stay in registers

constexpr size_t PACKED_HEADER_BYTES = 256;   // a packed buffer starts with its d2dmoe_packed_desc (64 bytes, padded)
constexpr int MD_BM = 64;       // tokens per workgroup of the dense sweep
constexpr int MD_HC = 256;      // hidden neurons per chunk (4 waves x 64) at D = 768
// ... and at any width the sweep is built for: 128 where the x tile leaves no room for a 256-neuron h tile
__host__ __device__ constexpr int sweep_chunk(int d_model) { return d_model <= 768 ? 256 : 128; }
constexpr int MD_WAVES = 4;
constexpr int MD_KS2 = MD_HC / 16;  // K=16 steps of the second GEMM per chunk
constexpr int MD_MAX_CHUNKS = 32;   // chunks per layer the dense sweep stages tables for (hidden <= 8192)
constexpr int MD_RING = 32;     // weight fragments kept in flight per wave (16 bytes per lane each)
constexpr int SP_MAX_MEAN_K = 8;    // the expert-major path is provisioned for at most N * 8 routed pairs
constexpr int SP_MAX_MEAN_K_GATED = 32;   // ... N * 32 for gated experts (up to 16 384 tokens)
constexpr int SP_GATED_MIN_PAIRS_PER_EXPERT = 128;   // ... and never fewer than E * 128 for gated experts
constexpr int SP_SEG = 32;          // tokens per plan segment (one wave): the tile of the fused router kernel
constexpr int MID_MAX_MEAN_K = 48;  // the compacted two-kernel path is provisioned for at most N * 48 routed pairs
constexpr int MID_HROW = 32;        // hidden values kept per routed pair (experts of at most 32 neurons), bf16

// Sections of the buffer d2dmoe_pack_weights writes.  A section is present when its kernel covers the shape.
struct PackedLayout {
  int hidden;      // E * Ed
  int n_chunks;    // ceil(hidden / sweep_chunk(D))
  int hidden_pad;  // n_chunks * sweep_chunk(D)
  int pieces;      // weight fragments per (wave, chunk) of the dense stream
  int nt;          // 32-neuron row tiles per expert in the expert-major section: ceil(Ed / 32)
  size_t w_off, b1_off, eidx_off;        // dense sweep: weight stream, bias (bf16), expert index per neuron (uint8)
  size_t r1_off, r2_off;                 // router fragments
  size_t s1_off, s2_off, sb_off;         // expert-major: W1 fragments, W2^T fragments, bias (bf16, padded to nt*32)
  size_t su_off;                         // expert-major, gated experts: fragments of the up projection
  size_t dc_off;                         // small-batch (decode) section
  size_t gm_off;                         // large-batch gated section (tiled products)
  size_t m1_off, m2_off;                 // compacted two-kernel path: W1 and W2^T fragments of the 16x16x32 MFMA
  size_t total;
  bool has_dense, has_router, has_sparse, has_decode, has_gemm, has_mid;
};
PackedLayout packed_layout(const d2dmoe_shape& sh);
int device_cu_count();
size_t mfma_decode_packed_bytes(const d2dmoe_shape& sh);
hipError_t launch_decode_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                              void* packed_section, hipStream_t s);
hipError_t launch_sparse_pack(const d2dmoe_shape& sh, const PackedLayout& L, const void* w1, const void* b1, const void* w2,
                              const void* w_up, void* packed, hipStream_t s);

// Per-segment routed-token counts and their per-expert prefix over segments (plan passes 1 and 2 of the expert-major
// paths): seg_counts[seg][e], seg_pairs[seg], then seg_offsets[seg][e] and totals[e].
void launch_plan_count_scan(const void* routing, int64_t N, int E, int32_t* seg_counts, int32_t* seg_pairs,
                            int32_t* seg_offsets, int32_t* totals, hipStream_t s, bool counts_ready = false);
hipError_t launch_mid_pack(const d2dmoe_shape& sh, const PackedLayout& L, const void* w1, const void* w2, void* packed,
                           hipStream_t s);

// two float32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ inline uint32_t pack2_bf16(float lo, float hi) {
  const f32x2 v = {lo, hi};
  const bf16x2 b = __builtin_convertvector(v, bf16x2);
  uint32_t u;
  __builtin_memcpy(&u, &b, 4);
  return u;
}

template <> __device__ inline uint32_t pack2_16<bf16_t>(float lo, float hi) { return pack2_bf16(lo, hi); }
template <> __device__ inline uint32_t pack2_16<f16_t>(float lo, float hi) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f16x2 h = {(_Float16)lo, (_Float16)hi};   // round-to-nearest-even each
  uint32_t u;
  __builtin_memcpy(&u, &h, 4);
  return u;
}

// 16-bit storage of the MFMA kernels that take both: bf16 (F16 = false) or IEEE half (F16 = true).  Fragment layouts are
// the same; what differs is the MFMA instruction, the decoding of stored values and the final rounding.
template <bool F16> __device__ __forceinline__ float dec16(uint32_t bits16) {       // low 16 bits -> float
  if constexpr (F16) { _Float16 h; const uint16_t u = (uint16_t)bits16; __builtin_memcpy(&h, &u, 2); return (float)h; }
  else return __uint_as_float(bits16 << 16);
}
template <bool F16> __device__ __forceinline__ float dec16_hi(uint32_t word) {      // high 16 bits -> float
  if constexpr (F16) return dec16<true>(word >> 16);
  else return __uint_as_float(word & 0xffff0000u);
}
template <bool F16> __device__ __forceinline__ uint32_t enc16x2(float lo, float hi) {
  if constexpr (F16) return pack2_16<f16_t>(lo, hi);
  else return pack2_bf16(lo, hi);
}
template <bool F16> __device__ __forceinline__ f32x16 mfma_32x32x16(const bf16x8& a, const bf16x8& b, const f32x16& c) {
  if constexpr (F16) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
}

template <bool F16> __device__ __forceinline__ f32x4_t mfma_16x16x32(const bf16x8& a, const bf16x8& b, const f32x4_t& c) {
  if constexpr (F16) {
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
}
// one value: rounded to the storage type (bits), and rounded and decoded again
template <bool F16> __device__ __forceinline__ uint16_t enc16(float v) { return (uint16_t)(enc16x2<F16>(v, 0.f) & 0xffffu); }
template <bool F16> __device__ __forceinline__ float round16(float v) { return dec16<F16>(enc16x2<F16>(v, 0.f) & 0xffffu); }
// LDS-only workgroup barrier: waits for this wave's LDS operations, not for its outstanding global loads.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// compile-time loop: f(std::integral_constant<int, I>) for I in [I0, N) -- indices stay constants without relying on
// the loop unroller
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

}  // namespace d2dmoe
