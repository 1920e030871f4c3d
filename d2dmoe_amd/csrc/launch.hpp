// Host-side launcher declarations shared between the kernel translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/d2dmoe.h"

namespace d2dmoe {

// ---- generic kernels (kernels_generic.hip) ----
template <typename T>
hipError_t launch_linear_act(const void* A, const void* B, void* C, int64_t M, int K, int Nout, int act, hipStream_t s);
bool linear_mfma_f32_supported(int64_t M, int K, int Nout);
hipError_t launch_linear_mfma_f32(const void* A, const void* B, void* C, int64_t M, int K, int Nout, int act, hipStream_t s);
// float16 storage on the matrix cores: K a multiple of 64, Nout a multiple of 32
bool linear_mfma_f16_supported(int64_t M, int K, int Nout);
hipError_t launch_linear_mfma_f16(const void* A, const void* B, void* C, int64_t M, int K, int Nout, int act, hipStream_t s);

hipError_t launch_fill_i32(int32_t* p, int64_t n, int32_t v, hipStream_t s);

template <typename T>
hipError_t launch_select(const void* norms, void* routing, int32_t* counts, int64_t N, int E, float thr_scale,
                         hipStream_t s);

size_t perm_workspace_bytes(int64_t N, int E);

template <typename T>
hipError_t launch_build_permutation(const void* routing, int64_t N, int E, int32_t* offsets, int32_t* token_idx,
                                    int64_t* sort_indices, int64_t* unsort_indices, int64_t* bincounts,
                                    void* workspace, hipStream_t s);

bool experts_generic_supported(const d2dmoe_shape& sh);

template <typename T>
hipError_t launch_experts_generic(const d2dmoe_shape& sh, const void* x, const void* routing, const void* w1,
                                  const void* b1, const void* w2, const void* w_up, const void* last_bias, void* out,
                                  hipStream_t s);

// ---- bf16 MFMA kernels (kernels_mfma.hip) ----
bool mfma_dense_supported(const d2dmoe_shape& sh);
bool mfma_sparse_falls_back_to_sweep(const d2dmoe_shape& sh);   // else: to the tiled products
bool mfma_router_supported(const d2dmoe_shape& sh);
size_t mfma_packed_bytes(const d2dmoe_shape& sh);
unsigned mfma_packed_sections(const d2dmoe_shape& sh);   // D2DMOE_SECTION_* bits of the buffer packed for sh
hipError_t launch_pack_header(const d2dmoe_packed_desc& d, void* packed, hipStream_t s);
hipError_t launch_mfma_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            const void* router_w1, const void* router_w2, void* packed, hipStream_t s);
// seg_counts / seg_pairs (optional): where the expert-major plan keeps its per-segment counts; written by the router
// kernel itself iff mfma_router_writes_plan_counts(sh), which saves that plan its first pass.
bool mfma_router_writes_plan_counts(const d2dmoe_shape& sh);
hipError_t launch_mfma_router_select(const d2dmoe_shape& sh, const void* x, const void* packed, void* routing,
                                     void* norms_out, int32_t* counts, float thr_scale, hipStream_t s,
                                     int32_t* seg_counts = nullptr, int32_t* seg_pairs = nullptr);
// With few tokens the sweep deals each tile's chunks to several workgroups and needs mfma_dense_workspace_bytes() of
// workspace for their float32 sums (without it, or with skip_flag, it runs one workgroup per tile).
size_t mfma_dense_workspace_bytes(const d2dmoe_shape& sh);
hipError_t launch_mfma_dense(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                             const void* last_bias, void* out, const int* skip_flag, void* workspace, size_t workspace_bytes,
                             hipStream_t s);
// the D = 1024 instances of the same sweep (kernels_dense_wide.hip)
hipError_t launch_mfma_dense_wide(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                                  const void* last_bias, void* out, const int* skip_flag, void* workspace,
                                  size_t workspace_bytes, hipStream_t s);
// out = round(sum over splits (ascending) of partial[split] + last_bias (+ x)); partial is [n_splits][N][D] float32
hipError_t launch_sum_partials(const float* partial, const void* last_bias, const void* x, void* out, int64_t N, int D,
                               int n_splits, int add_residual, hipStream_t s, int dtype = D2DMOE_BF16, const int* skip_flag = nullptr);

// ---- bf16 MFMA expert-major path (kernels_sparse.hip) ----
bool mfma_sparse_supported(const d2dmoe_shape& sh);
size_t mfma_sparse_workspace_bytes(const d2dmoe_shape& sh);
int mfma_sparse_capacity_k(const d2dmoe_shape& sh);   // routed pairs per token the path is provisioned for
int64_t mfma_sparse_capacity_pairs(const d2dmoe_shape& sh);   // ... and in all, for this number of tokens
// Offset inside the expert-major workspace at which a gated layer's fall-back (the tiled products) may work: behind the
// plan, in the region the per-pair rows would have used.
size_t mfma_sparse_fallback_offset(const d2dmoe_shape& sh);
// Plans the call on the device (permutation, tiles, path flag), runs the expert-major kernels when the number of routed
// pairs is at most n_tokens * max_mean_k, and leaves *flag == 0 otherwise so that the dense sweep (launched by the
// caller with skip_flag = the returned pointer) does the work instead.
// counts_ready: the per-segment counts are already in the workspace (mfma_sparse_plan_counts names the place).
hipError_t launch_mfma_sparse(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                              const void* last_bias, void* out, void* workspace, int max_mean_k, const int** flag_out,
                              hipStream_t s, bool counts_ready = false);
void mfma_sparse_plan_counts(const d2dmoe_shape& sh, void* workspace, int32_t** seg_counts, int32_t** seg_pairs);
// ---- compacted two-kernel bf16 MFMA path for middling routing density (kernels_mid.hip) ----
bool mfma_mid_supported(const d2dmoe_shape& sh);
size_t mfma_mid_workspace_bytes(const d2dmoe_shape& sh);
int64_t mfma_mid_capacity_pairs(const d2dmoe_shape& sh);
// Plans on the device and runs the two kernels when the routed pairs fit the capacity; otherwise *flag stays 0 and the
// caller's dense sweep (skip_flag = the returned pointer) does the work.
hipError_t launch_mfma_mid(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed,
                           const void* last_bias, void* out, void* workspace, const int** flag_out, hipStream_t s);
// ---- small-batch (<= 16 tokens) bf16 MFMA path (kernels_decode.hip) ----
bool mfma_decode_supported(const d2dmoe_shape& sh);
size_t mfma_decode_workspace_bytes(const d2dmoe_shape& sh);
hipError_t launch_mfma_decode(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                              const void* last_bias, void* out, void* workspace, hipStream_t s);
size_t mfma_decode_section_offset(const d2dmoe_shape& sh);
bool linear_skinny_supported(int64_t N, int K, int dtype);
hipError_t launch_linear_skinny(const void* A, const void* B, void* C, int N, int K, int Nout, int act, hipStream_t s,
                                int dtype = D2DMOE_BF16);
// whole layer for at most 16 tokens in three launches (router included; the routing is derived inside the output kernel)
bool mfma_decode_layer_supported(const d2dmoe_shape& sh);
hipError_t launch_mfma_decode_layer(const d2dmoe_shape& sh, const void* x, const void* router_w1, const void* router_w2,
                                    float thr_scale, const void* packed_section, const void* last_bias, void* router_hidden,
                                    void* norms, void* routing, int32_t* counts, void* out, void* workspace, hipStream_t s);
// ---- two tiled bf16 MFMA products with the hidden activations in the workspace (kernels_gemm.hip) ----
bool mfma_gemm_supported(const d2dmoe_shape& sh);
size_t mfma_gemm_packed_bytes(const d2dmoe_shape& sh);
size_t mfma_gemm_workspace_bytes(const d2dmoe_shape& sh);
size_t mfma_gemm_section_offset(const d2dmoe_shape& sh);
hipError_t launch_gemm_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, const void* w_up,
                            void* packed_section, hipStream_t s);
hipError_t launch_mfma_gemm(const d2dmoe_shape& sh, const void* x, const void* routing, const void* packed_section,
                            const void* last_bias, void* out, void* workspace, hipStream_t s, const int* skip_flag = nullptr);
void launch_perm_scan(const int32_t* seg_counts, int32_t* seg_offsets, int32_t* totals, int E, int64_t n_seg, hipStream_t s);

// ---- per-expert output norms, the router-training targets (kernels_norms.hip) ----
bool mfma_norms_supported(const d2dmoe_shape& sh);
size_t mfma_norms_packed_bytes(const d2dmoe_shape& sh);
hipError_t launch_norms_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, void* packed, hipStream_t s);
hipError_t launch_mfma_norms(const d2dmoe_shape& sh, const void* x, const void* packed, void* norms, hipStream_t s);

}  // namespace d2dmoe
