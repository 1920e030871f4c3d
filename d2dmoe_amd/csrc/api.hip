// C ABI of the MoE-FFN forward path (declared in include/d2dmoe.h): argument checks and kernel sequencing.
// Nothing here allocates, synchronises or reads device memory on the host.
#include <hip/hip_runtime.h>

#include <mutex>

#include "common.hpp"
#include "launch.hpp"

using namespace d2dmoe;

// Workspace of d2dmoe_forward_static: one array per GPU, part of the loaded code object, held until the process ends.
// Host code never uses this name as an address -- it is a host-side stand-in; the device address is looked up once per
// device with hipGetSymbolAddress and kept in static_scratch_ptr[].
static __device__ __align__(256) unsigned char scratch[D2DMOE_STATIC_WORKSPACE_BYTES];

// Keeps the array in the device code object whatever the optimiser thinks of a variable no other kernel names.
__global__ void static_scratch_anchor_kernel(int v) { scratch[0] = (unsigned char)v; }

namespace {

constexpr int kMaxDevices = 64;
void* static_scratch_ptr[kMaxDevices] = {};
std::mutex static_scratch_mutex;

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return D2DMOE_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(static_scratch_mutex);
  if (static_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr || (((uintptr_t)p) & 255u)) return D2DMOE_E_WORKSPACE;
    static_scratch_ptr[dev] = p;
  }
  *out = static_scratch_ptr[dev];
  return D2DMOE_OK;
}

inline size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }
inline size_t elem_size(int dtype) { return dtype == D2DMOE_F32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype == D2DMOE_F32 || dtype == D2DMOE_BF16 || dtype == D2DMOE_F16; }
inline bool act_ok(int a) { return a >= D2DMOE_ACT_RELU && a <= D2DMOE_ACT_ABS; }
inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

int check_shape(const d2dmoe_shape* sh) {
  if (sh == nullptr) return D2DMOE_E_NULL;
  if (!dtype_ok(sh->dtype)) return D2DMOE_E_DTYPE;
  if (!act_ok(sh->activation) || !act_ok(sh->router_activation) || !act_ok(sh->router_output_activation))
    return D2DMOE_E_ACTIVATION;
  if (sh->n_tokens < 0 || sh->d_model <= 0 || sh->n_experts <= 0 || sh->expert_dim <= 0) return D2DMOE_E_SHAPE;
  if (sh->n_experts > 1024) return D2DMOE_E_SHAPE;
  if (sh->n_tokens > (int64_t)1 << 31) return D2DMOE_E_SHAPE;
  if (sh->n_tokens * (int64_t)sh->n_experts >= ((int64_t)1 << 31)) return D2DMOE_E_SHAPE;  // pair indices are int32
  return D2DMOE_OK;
}

// The descriptor d2dmoe_pack_weights hands out for a buffer packed for sh.
d2dmoe_packed_desc make_packed_desc(const d2dmoe_shape& sh) {
  d2dmoe_packed_desc d = {};
  d.magic = D2DMOE_PACKED_MAGIC;
  d.layout_version = D2DMOE_PACKED_LAYOUT_VERSION;
  d.dtype = sh.dtype; d.d_model = sh.d_model; d.n_experts = sh.n_experts; d.expert_dim = sh.expert_dim;
  d.gated = sh.gated ? 1 : 0;
  d.router_width = mfma_router_supported(sh) ? sh.router_width : 0;
  d.sections = mfma_packed_sections(sh);
  d.bytes = mfma_packed_bytes(sh);
  return d;
}

// Host-side check of a packed buffer's descriptor against the shape of the call that is about to use it.  need_router:
// the call runs the fused router kernel out of the buffer's router section.
int check_packed(const d2dmoe_shape& sh, const void* packed, const d2dmoe_packed_desc* d, bool need_router) {
  if (packed == nullptr) return D2DMOE_OK;
  if (d == nullptr) return D2DMOE_E_PACKED;
  if (d->magic != D2DMOE_PACKED_MAGIC || d->layout_version != D2DMOE_PACKED_LAYOUT_VERSION) return D2DMOE_E_PACKED;
  if (d->dtype != sh.dtype || d->d_model != sh.d_model || d->n_experts != sh.n_experts || d->expert_dim != sh.expert_dim ||
      d->gated != (sh.gated ? 1 : 0))
    return D2DMOE_E_PACKED;
  // what a buffer packed for this layer with the router width the descriptor names looks like (the router section is
  // the last one, so the other sections do not move with it)
  d2dmoe_shape as_packed = sh;
  as_packed.router_width = d->router_width;
  if (d->router_width > 0) {   // packed with a router section: the fused router kernel's own activations
    as_packed.router_activation = D2DMOE_ACT_RELU;
    as_packed.router_output_activation = D2DMOE_ACT_ABS;
  }
  const d2dmoe_packed_desc want = make_packed_desc(as_packed);
  if (want.bytes == 0 || d->bytes != want.bytes || d->sections != want.sections || want.router_width != d->router_width)
    return D2DMOE_E_PACKED;
  if (need_router && (!(d->sections & D2DMOE_SECTION_ROUTER) || d->router_width != sh.router_width)) return D2DMOE_E_PACKED;
  return D2DMOE_OK;
}

struct ForwardWorkspace {
  size_t hidden_off, norms_off, perm_off, total;
};

ForwardWorkspace plan_workspace(const d2dmoe_shape& sh) {
  ForwardWorkspace w;
  const size_t es = elem_size(sh.dtype);
  const size_t N = (size_t)sh.n_tokens;
  size_t off = 0;
  w.hidden_off = off; off += align_up(N * (size_t)(sh.router_width > 0 ? sh.router_width : 0) * es);
  w.norms_off = off;  off += align_up(N * (size_t)sh.n_experts * es);
  size_t scratch = perm_workspace_bytes(sh.n_tokens, sh.n_experts);
  const size_t sparse = mfma_sparse_workspace_bytes(sh);   // plan + result rows of the expert-major path
  if (sparse > scratch) scratch = sparse;
  const size_t decode = mfma_decode_workspace_bytes(sh);   // hidden fragments + expert flags of the small-batch path
  if (decode > scratch) scratch = decode;
  const size_t dsplit = mfma_dense_workspace_bytes(sh);    // float32 sums of the chunk-split dense sweep (few tokens)
  if (dsplit > scratch) scratch = dsplit;
  const size_t gemm = (sh.n_tokens > 16) ? mfma_gemm_workspace_bytes(sh) : 0;   // H fragments + partial sums of the gated path
  if (gemm > scratch) scratch = gemm;
  const size_t mid = (sh.n_tokens > 16) ? mfma_mid_workspace_bytes(sh) : 0;     // plan + hidden rows of the compacted path
  if (mid > scratch) scratch = mid;
  w.perm_off = off;   off += align_up(scratch);
  w.total = off;
  return w;
}

}  // namespace

extern "C" {

int d2dmoe_version(void) { return D2DMOE_VERSION; }

const char* d2dmoe_status_string(int status) {
  switch (status) {
    case D2DMOE_OK: return "ok";
    case D2DMOE_E_NULL: return "a required pointer is NULL";
    case D2DMOE_E_SHAPE: return "size non-positive or outside the supported range";
    case D2DMOE_E_DTYPE: return "unknown element type";
    case D2DMOE_E_ACTIVATION: return "unknown activation";
    case D2DMOE_E_WORKSPACE: return "workspace missing, misaligned or too small";
    case D2DMOE_E_UNSUPPORTED: return "no kernel for this request in this build";
    case D2DMOE_E_ALIGN: return "tensor pointer not aligned to 16 bytes";
    case D2DMOE_E_STATIC_LIMIT: return "shape needs more workspace than the static array of d2dmoe_forward_static holds";
    case D2DMOE_E_PACKED: return "packed buffer without its descriptor, or packed for another layer or layout version";
    default: break;
  }
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "unknown status";
}

size_t d2dmoe_workspace_bytes(const d2dmoe_shape* shape) {
  if (check_shape(shape) != D2DMOE_OK) return 0;
  return plan_workspace(*shape).total;
}

int d2dmoe_router(const void* x, const void* router_w1, const void* router_w2, void* norms, int64_t n_tokens,
                  int32_t d_model, int32_t router_width, int32_t n_experts, int32_t dtype, int32_t activation,
                  int32_t output_activation, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !router_w1 || !router_w2 || !norms) return D2DMOE_E_NULL;
  if (!dtype_ok(dtype)) return D2DMOE_E_DTYPE;
  if (!act_ok(activation) || !act_ok(output_activation)) return D2DMOE_E_ACTIVATION;
  if (n_tokens < 0 || d_model <= 0 || router_width <= 0 || n_experts <= 0) return D2DMOE_E_SHAPE;
  if (n_tokens == 0) return D2DMOE_OK;
  const size_t need = (size_t)n_tokens * router_width * elem_size(dtype);
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return D2DMOE_E_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  hipError_t e;
  if (linear_skinny_supported(n_tokens, d_model, dtype) && linear_skinny_supported(n_tokens, router_width, dtype)) {
    // a handful of tokens: MFMA kernels that spread the output features over the machine
    e = launch_linear_skinny(x, router_w1, workspace, (int)n_tokens, d_model, router_width, activation, s, dtype);
    if (e == hipSuccess)
      e = launch_linear_skinny(workspace, router_w2, norms, (int)n_tokens, router_width, n_experts, output_activation, s, dtype);
  } else if (dtype == D2DMOE_F32) {
    // float32 on the matrix cores where the widths allow 16-byte operand loads and whole 32-column tiles
    const bool m1 = linear_mfma_f32_supported(n_tokens, d_model, router_width) && aligned16(x) && aligned16(router_w1);
    const bool m2 = linear_mfma_f32_supported(n_tokens, router_width, n_experts) && aligned16(router_w2);
    e = m1 ? launch_linear_mfma_f32(x, router_w1, workspace, n_tokens, d_model, router_width, activation, s)
           : launch_linear_act<float>(x, router_w1, workspace, n_tokens, d_model, router_width, activation, s);
    if (e == hipSuccess)
      e = m2 ? launch_linear_mfma_f32(workspace, router_w2, norms, n_tokens, router_width, n_experts, output_activation, s)
             : launch_linear_act<float>(workspace, router_w2, norms, n_tokens, router_width, n_experts, output_activation, s);
  } else if (dtype == D2DMOE_F16) {
    const bool m1 = linear_mfma_f16_supported(n_tokens, d_model, router_width) && aligned16(x) && aligned16(router_w1);
    const bool m2 = linear_mfma_f16_supported(n_tokens, router_width, n_experts) && aligned16(router_w2);
    e = m1 ? launch_linear_mfma_f16(x, router_w1, workspace, n_tokens, d_model, router_width, activation, s)
           : launch_linear_act<f16_t>(x, router_w1, workspace, n_tokens, d_model, router_width, activation, s);
    if (e == hipSuccess)
      e = m2 ? launch_linear_mfma_f16(workspace, router_w2, norms, n_tokens, router_width, n_experts, output_activation, s)
             : launch_linear_act<f16_t>(workspace, router_w2, norms, n_tokens, router_width, n_experts, output_activation, s);
  } else {
    e = launch_linear_act<bf16_t>(x, router_w1, workspace, n_tokens, d_model, router_width, activation, s);
    if (e == hipSuccess) e = launch_linear_act<bf16_t>(workspace, router_w2, norms, n_tokens, router_width, n_experts, output_activation, s);
  }
  return (int)e;
}

int d2dmoe_select(const void* norms, void* routing, int32_t* counts, int64_t n_tokens, int32_t n_experts,
                  int32_t dtype, float thr_scale, void* stream) {
  if (!norms || !routing) return D2DMOE_E_NULL;
  if (!dtype_ok(dtype)) return D2DMOE_E_DTYPE;
  if (n_tokens < 0 || n_experts <= 0 || n_experts > 1024) return D2DMOE_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (n_tokens == 0) {
    if (counts) return (int)launch_fill_i32(counts, n_experts, 0, s);
    return D2DMOE_OK;
  }
  if (dtype == D2DMOE_F16) return (int)launch_select<f16_t>(norms, routing, counts, n_tokens, n_experts, thr_scale, s);
  hipError_t e = (dtype == D2DMOE_F32) ? launch_select<float>(norms, routing, counts, n_tokens, n_experts, thr_scale, s)
                                       : launch_select<bf16_t>(norms, routing, counts, n_tokens, n_experts, thr_scale, s);
  return (int)e;
}

int d2dmoe_build_permutation(const void* routing, int64_t n_tokens, int32_t n_experts, int32_t dtype,
                             int32_t* offsets, int32_t* token_idx, int64_t* sort_indices, int64_t* unsort_indices,
                             int64_t* bincounts, void* workspace, size_t workspace_bytes, void* stream) {
  if (!offsets || !token_idx) return D2DMOE_E_NULL;
  if (!dtype_ok(dtype)) return D2DMOE_E_DTYPE;
  if (n_tokens < 0 || n_experts <= 0 || n_experts > 1024) return D2DMOE_E_SHAPE;
  if (n_tokens * (int64_t)n_experts >= ((int64_t)1 << 31)) return D2DMOE_E_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (n_tokens == 0) {
    hipError_t e = launch_fill_i32(offsets, n_experts + 1, 0, s);
    if (e == hipSuccess && bincounts) e = launch_fill_i32((int32_t*)bincounts, 2 * (int64_t)n_experts, 0, s);
    return (int)e;
  }
  if (!routing) return D2DMOE_E_NULL;
  if (!workspace || workspace_bytes < perm_workspace_bytes(n_tokens, n_experts) || !aligned16(workspace))
    return D2DMOE_E_WORKSPACE;
  if (dtype == D2DMOE_F16)
    return (int)launch_build_permutation<f16_t>(routing, n_tokens, n_experts, offsets, token_idx, sort_indices, unsort_indices,
                                                bincounts, workspace, s);
  hipError_t e = (dtype == D2DMOE_F32)
                     ? launch_build_permutation<float>(routing, n_tokens, n_experts, offsets, token_idx, sort_indices,
                                                       unsort_indices, bincounts, workspace, s)
                     : launch_build_permutation<bf16_t>(routing, n_tokens, n_experts, offsets, token_idx, sort_indices,
                                                        unsort_indices, bincounts, workspace, s);
  return (int)e;
}

size_t d2dmoe_packed_bytes(const d2dmoe_shape* shape) {
  if (check_shape(shape) != D2DMOE_OK) return 0;
  if (!mfma_dense_supported(*shape) && !mfma_router_supported(*shape) && !mfma_decode_supported(*shape) &&
      !mfma_gemm_supported(*shape)) return 0;
  return mfma_packed_bytes(*shape);
}

int d2dmoe_packed_describe(const d2dmoe_shape* shape, d2dmoe_packed_desc* desc) {
  const int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  if (!desc) return D2DMOE_E_NULL;
  if (mfma_packed_bytes(*shape) == 0) return D2DMOE_E_UNSUPPORTED;
  *desc = make_packed_desc(*shape);
  return D2DMOE_OK;
}

int d2dmoe_packed_desc_from_header(const void* host_header_64_bytes, d2dmoe_packed_desc* desc) {
  if (!host_header_64_bytes || !desc) return D2DMOE_E_NULL;
  d2dmoe_packed_desc d;
  __builtin_memcpy(&d, host_header_64_bytes, sizeof(d));
  if (d.magic != D2DMOE_PACKED_MAGIC) return D2DMOE_E_PACKED;
  *desc = d;
  return D2DMOE_OK;
}

int d2dmoe_pack_weights(const d2dmoe_shape* shape, const void* w1, const void* b1, const void* w2, const void* w_up,
                        const void* router_w1, const void* router_w2, void* packed, size_t packed_bytes,
                        d2dmoe_packed_desc* desc_out, void* stream) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  if (!w1 || !w2 || !packed || !desc_out) return D2DMOE_E_NULL;
  if (!mfma_dense_supported(*shape) && !mfma_router_supported(*shape) && !mfma_decode_supported(*shape) &&
      !mfma_gemm_supported(*shape))
    return D2DMOE_E_UNSUPPORTED;
  if (shape->gated && !w_up) return D2DMOE_E_NULL;
  if (mfma_router_supported(*shape) && (!router_w1 || !router_w2)) return D2DMOE_E_NULL;
  if (packed_bytes < mfma_packed_bytes(*shape) || (((uintptr_t)packed) & 255u)) return D2DMOE_E_WORKSPACE;
  const d2dmoe_packed_desc d = make_packed_desc(*shape);
  hipError_t e = launch_pack_header(d, packed, (hipStream_t)stream);
  if (e == hipSuccess) e = launch_mfma_pack(*shape, w1, b1, w2, w_up, router_w1, router_w2, packed, (hipStream_t)stream);
  if (e == hipSuccess) *desc_out = d;
  return (int)e;
}

// plan_counts_ready: the router kernel of this call has already left the expert-major plan's per-segment counts in
// the workspace (d2dmoe_forward only)
static int experts_impl(const d2dmoe_shape* shape, const void* x, const void* routing, const void* w1, const void* b1,
                        const void* w2, const void* w_up, const void* last_bias, const void* packed,
                        const d2dmoe_packed_desc* packed_desc, void* out, int32_t path, void* workspace,
                        size_t workspace_bytes, void* stream, bool plan_counts_ready) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  const d2dmoe_shape& sh = *shape;
  st = check_packed(sh, packed, packed_desc, false);
  if (st != D2DMOE_OK) return st;
  if (sh.n_tokens == 0) return D2DMOE_OK;
  if (!x || !routing || !w1 || !w2 || !out) return D2DMOE_E_NULL;
  if (sh.gated && !w_up) return D2DMOE_E_NULL;
  if (sh.gated && b1) return D2DMOE_E_UNSUPPORTED;
  if (!sh.gated && w_up) return D2DMOE_E_SHAPE;
  if (!aligned16(x) || !aligned16(out) || !aligned16(routing)) return D2DMOE_E_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (path == D2DMOE_PATH_AUTO) {
    // the small-batch kernels take 16 tokens per pass; gated experts (bound by the weight stream up to a few hundred
    // tokens) are worth up to three passes
    if (packed != nullptr && sh.n_tokens <= (sh.gated ? 48 : 16) && mfma_decode_supported(sh)) path = D2DMOE_PATH_MFMA_DECODE;
    else if (packed != nullptr && sh.gated && sh.n_tokens <= 128 && mfma_sparse_supported(sh) && mfma_gemm_supported(sh))
      path = D2DMOE_PATH_MFMA_SPARSE;   // still bound by the weight stream: expert-major whatever the routing
    // big experts: the dense sweep cannot skip anything (a chunk of 256 neurons is two experts), so the expert-major
    // path is tried whatever the threshold; it hands over to the sweep on the device when the routing is dense
    else if (packed != nullptr && !sh.gated && sh.expert_dim > 64 && mfma_sparse_supported(sh) && mfma_sparse_falls_back_to_sweep(sh) &&
             workspace != nullptr && workspace_bytes >= mfma_sparse_workspace_bytes(sh))
      path = D2DMOE_PATH_MFMA_SPARSE;
    else if (packed != nullptr && mfma_dense_supported(sh)) path = D2DMOE_PATH_MFMA_DENSE;
    else if (packed != nullptr && mfma_gemm_supported(sh)) path = D2DMOE_PATH_MFMA_GEMM;
    else path = D2DMOE_PATH_GENERIC;
  }
  switch (path) {
    case D2DMOE_PATH_GENERIC: {
      if (!experts_generic_supported(sh)) return D2DMOE_E_UNSUPPORTED;
      if (sh.dtype == D2DMOE_F16)
        return (int)launch_experts_generic<f16_t>(sh, x, routing, w1, b1, w2, w_up, last_bias, out, s);
      hipError_t e = (sh.dtype == D2DMOE_F32)
                         ? launch_experts_generic<float>(sh, x, routing, w1, b1, w2, w_up, last_bias, out, s)
                         : launch_experts_generic<bf16_t>(sh, x, routing, w1, b1, w2, w_up, last_bias, out, s);
      return (int)e;
    }
    case D2DMOE_PATH_MFMA_DENSE: {
      if (!mfma_dense_supported(sh)) return D2DMOE_E_UNSUPPORTED;
      if (!packed) return D2DMOE_E_NULL;
      return (int)launch_mfma_dense(sh, x, routing, packed, last_bias, out, nullptr, workspace, workspace_bytes, s);
    }
    case D2DMOE_PATH_MFMA_SPARSE: {
      // expert-major when the routed pairs fit the provisioned capacity, else the dense sweep: decided on the device
      if (!mfma_sparse_supported(sh)) return D2DMOE_E_UNSUPPORTED;
      // the fall-back: the dense sweep (ungated, D = 768 or 1024, up to 256 experts), else the tiled products
      const bool fb_gemm = !mfma_sparse_falls_back_to_sweep(sh);
      if (fb_gemm && !mfma_gemm_supported(sh)) return D2DMOE_E_UNSUPPORTED;
      if (!packed) return D2DMOE_E_NULL;
      const size_t need = mfma_sparse_workspace_bytes(sh);
      if (!workspace || workspace_bytes < need || (((uintptr_t)workspace) & 255u)) return D2DMOE_E_WORKSPACE;
      // the tiled products of the fall-back work behind the plan: they must fit what is left there
      if (fb_gemm && sh.n_tokens * (int64_t)sh.n_experts > mfma_sparse_capacity_pairs(sh) &&
          workspace_bytes < mfma_sparse_fallback_offset(sh) + mfma_gemm_workspace_bytes(sh))
        return D2DMOE_E_WORKSPACE;
      const int* flag = nullptr;
      hipError_t e = launch_mfma_sparse(sh, x, routing, packed, last_bias, out, workspace, mfma_sparse_capacity_k(sh), &flag, s,
                                        plan_counts_ready);
      if (e != hipSuccess) return (int)e;
      // with every expert routed to by every token the pairs still fit: the fall-back can never be needed
      if (sh.n_tokens * (int64_t)sh.n_experts <= mfma_sparse_capacity_pairs(sh)) return D2DMOE_OK;
      if (fb_gemm)   // the tiled products work behind the plan in the same workspace
        return (int)launch_mfma_gemm(sh, x, routing, (const char*)packed + mfma_gemm_section_offset(sh), last_bias, out,
                                     (char*)workspace + mfma_sparse_fallback_offset(sh), s, flag);
      // (the sweep's split tail tiles leave their partial sums in the pair rows' region, idle when the sweep runs)
      const size_t fb_off = mfma_sparse_fallback_offset(sh);
      return (int)launch_mfma_dense(sh, x, routing, packed, last_bias, out, flag, (char*)workspace + fb_off,
                                    workspace_bytes - fb_off, s);
    }
    case D2DMOE_PATH_MFMA_MID: {
      // compacted two-kernel path when the routed pairs fit the provisioned capacity, else the dense sweep: decided on
      // the device
      if (!mfma_mid_supported(sh) || !mfma_sparse_falls_back_to_sweep(sh)) return D2DMOE_E_UNSUPPORTED;
      if (!packed) return D2DMOE_E_NULL;
      const size_t need = mfma_mid_workspace_bytes(sh);
      if (!workspace || workspace_bytes < need || (((uintptr_t)workspace) & 255u)) return D2DMOE_E_WORKSPACE;
      const int* flag = nullptr;
      hipError_t e = launch_mfma_mid(sh, x, routing, packed, last_bias, out, workspace, &flag, s);
      if (e != hipSuccess) return (int)e;
      if (sh.n_tokens * (int64_t)sh.n_experts <= mfma_mid_capacity_pairs(sh)) return D2DMOE_OK;   // always fits
      return (int)launch_mfma_dense(sh, x, routing, packed, last_bias, out, flag, nullptr, 0, s);
    }
    case D2DMOE_PATH_MFMA_DECODE: {
      if (!mfma_decode_supported(sh) || sh.n_tokens > 48) return D2DMOE_E_UNSUPPORTED;
      if (!packed) return D2DMOE_E_NULL;
      const size_t need = mfma_decode_workspace_bytes(sh);
      if (!workspace || workspace_bytes < need || (((uintptr_t)workspace) & 255u)) return D2DMOE_E_WORKSPACE;
      // passes of 16 tokens, one after the other on the stream, sharing the workspace
      const size_t es = elem_size(sh.dtype);
      for (int64_t t0 = 0; t0 < sh.n_tokens; t0 += 16) {
        d2dmoe_shape part = sh;
        part.n_tokens = (sh.n_tokens - t0 < 16) ? (sh.n_tokens - t0) : 16;
        const hipError_t e = launch_mfma_decode(part, (const char*)x + t0 * sh.d_model * es, (const char*)routing + t0 * sh.n_experts * es,
                                                (const char*)packed + mfma_decode_section_offset(sh), last_bias,
                                                (char*)out + t0 * sh.d_model * es, workspace, s);
        if (e != hipSuccess) return (int)e;
      }
      return D2DMOE_OK;
    }
    case D2DMOE_PATH_MFMA_GEMM: {
      if (!mfma_gemm_supported(sh)) return D2DMOE_E_UNSUPPORTED;
      if (!packed) return D2DMOE_E_NULL;
      const size_t need = mfma_gemm_workspace_bytes(sh);
      if (!workspace || workspace_bytes < need || (((uintptr_t)workspace) & 255u)) return D2DMOE_E_WORKSPACE;
      return (int)launch_mfma_gemm(sh, x, routing, (const char*)packed + mfma_gemm_section_offset(sh), last_bias, out,
                                   workspace, s);
    }
    default: return D2DMOE_E_UNSUPPORTED;
  }
}

int d2dmoe_experts(const d2dmoe_shape* shape, const void* x, const void* routing, const void* w1, const void* b1,
                   const void* w2, const void* w_up, const void* last_bias, const void* packed,
                   const d2dmoe_packed_desc* packed_desc, void* out, int32_t path, void* workspace, size_t workspace_bytes,
                   void* stream) {
  return experts_impl(shape, x, routing, w1, b1, w2, w_up, last_bias, packed, packed_desc, out, path, workspace,
                      workspace_bytes, stream, false);
}

// seg_counts / seg_pairs: see launch_mfma_router_select
static int router_select_impl(const d2dmoe_shape* shape, const void* x, const void* router_w1, const void* router_w2,
                              const void* packed, const d2dmoe_packed_desc* packed_desc, float thr_scale, void* norms_out,
                              void* routing, int32_t* counts, void* workspace, size_t workspace_bytes, void* stream,
                              int32_t* seg_counts, int32_t* seg_pairs) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  const d2dmoe_shape& sh = *shape;
  if (!routing) return D2DMOE_E_NULL;
  if (sh.router_width <= 0) return D2DMOE_E_SHAPE;
  // (a buffer packed without the router section is no error here: the call then runs the unfused router kernels)
  st = check_packed(sh, packed, packed_desc, false);
  if (st != D2DMOE_OK) return st;
  if (packed != nullptr && !((packed_desc->sections & D2DMOE_SECTION_ROUTER) && packed_desc->router_width == sh.router_width))
    packed = nullptr;
  if (sh.n_tokens == 0) return counts ? (int)launch_fill_i32(counts, sh.n_experts, 0, (hipStream_t)stream) : D2DMOE_OK;
  if (!x) return D2DMOE_E_NULL;
  if (packed != nullptr && mfma_router_supported(sh) && sh.n_tokens > 16) {
    if (!aligned16(x) || !aligned16(routing) || (norms_out && !aligned16(norms_out))) return D2DMOE_E_ALIGN;
    return (int)launch_mfma_router_select(sh, x, packed, routing, norms_out, counts, thr_scale, (hipStream_t)stream,
                                          seg_counts, seg_pairs);
  }
  if (!router_w1 || !router_w2) return D2DMOE_E_NULL;
  const ForwardWorkspace plan = plan_workspace(sh);
  if (!workspace || workspace_bytes < plan.total || (((uintptr_t)workspace) & 255u)) return D2DMOE_E_WORKSPACE;
  char* ws = (char*)workspace;
  void* nbuf = norms_out ? norms_out : (void*)(ws + plan.norms_off);
  st = d2dmoe_router(x, router_w1, router_w2, nbuf, sh.n_tokens, sh.d_model, sh.router_width, sh.n_experts, sh.dtype,
                     sh.router_activation, sh.router_output_activation, ws + plan.hidden_off,
                     plan.norms_off - plan.hidden_off, stream);
  if (st != D2DMOE_OK) return st;
  return d2dmoe_select(nbuf, routing, counts, sh.n_tokens, sh.n_experts, sh.dtype, thr_scale, stream);
}

int d2dmoe_router_select(const d2dmoe_shape* shape, const void* x, const void* router_w1, const void* router_w2,
                         const void* packed, const d2dmoe_packed_desc* packed_desc, float thr_scale, void* norms_out,
                         void* routing, int32_t* counts, void* workspace, size_t workspace_bytes, void* stream) {
  return router_select_impl(shape, x, router_w1, router_w2, packed, packed_desc, thr_scale, norms_out, routing, counts,
                            workspace, workspace_bytes, stream, nullptr, nullptr);
}

int d2dmoe_forward(const d2dmoe_shape* shape, const void* x, const void* router_w1, const void* router_w2,
                   float thr_scale, const void* w1, const void* b1, const void* w2, const void* w_up,
                   const void* last_bias, const void* packed, const d2dmoe_packed_desc* packed_desc, const void* norms_in,
                   void* norms_out, void* routing, int32_t* counts, void* out, int32_t path, void* workspace,
                   size_t workspace_bytes, void* stream) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  const d2dmoe_shape& sh = *shape;
  if (!routing || !out) return D2DMOE_E_NULL;
  st = check_packed(sh, packed, packed_desc, false);
  if (st != D2DMOE_OK) return st;
  if (sh.n_tokens == 0) return counts ? (int)launch_fill_i32(counts, sh.n_experts, 0, (hipStream_t)stream) : D2DMOE_OK;
  if (!x) return D2DMOE_E_NULL;
  const ForwardWorkspace plan = plan_workspace(sh);
  if (!workspace || workspace_bytes < plan.total || (((uintptr_t)workspace) & 255u)) return D2DMOE_E_WORKSPACE;
  char* ws = (char*)workspace;
  if (norms_in == nullptr && (path == D2DMOE_PATH_AUTO || path == D2DMOE_PATH_MFMA_DECODE) && packed != nullptr &&
      mfma_decode_layer_supported(sh) && router_w1 && router_w2 && w1 && w2 && (sh.gated ? (w_up && !b1) : !w_up) &&
      aligned16(x) && aligned16(out) && aligned16(routing) && aligned16(router_w1) && aligned16(router_w2) &&
      (!norms_out || aligned16(norms_out))) {
    // a handful of tokens: three launches for the whole layer, the router running beside the experts' first layer
    void* nbuf = norms_out ? norms_out : (void*)(ws + plan.norms_off);
    return (int)launch_mfma_decode_layer(sh, x, router_w1, router_w2, thr_scale,
                                         (const char*)packed + mfma_decode_section_offset(sh), last_bias, ws + plan.hidden_off,
                                         nbuf, routing, counts, out, ws + plan.perm_off, (hipStream_t)stream);
  }
  // A high threshold fraction keeps few experts per token: take the expert-major path (it falls back to the dense
  // sweep on the device if the routing turns out dense after all).
  // (gated experts, and ungated ones at widths other than 768: from a lower fraction on -- their capacity is 12 or 32
  // routed experts per token instead of 8, their dense alternative costs several times the expert-major path at few
  // experts per token, and the device-side switch is cheap next to it;
  // and with at most 128 tokens whatever the fraction -- the layer is bound by the weight stream there, which the tiled
  // products pay for with whole 256-token tiles;
  // big ungated experts from a lower fraction on, and whatever the fraction when the norms are handed in -- the
  // reference benchmark's Bernoulli override, where the fraction says nothing about the density: the dense sweep
  // cannot skip at their granularity)
  if (path == D2DMOE_PATH_AUTO && sh.n_tokens > (sh.gated && mfma_decode_supported(sh) ? 48 : 16) && packed != nullptr &&
      (thr_scale >= ((sh.d_model != 768 || !mfma_sparse_falls_back_to_sweep(sh)) ? 0.5f : 0.75f) || (sh.gated && sh.n_tokens <= 128) ||
       (!sh.gated && sh.expert_dim > 64 && (norms_in != nullptr || thr_scale >= 0.5f))) &&
      mfma_sparse_supported(sh) &&
      (mfma_sparse_falls_back_to_sweep(sh) || mfma_gemm_supported(sh)))
    path = D2DMOE_PATH_MFMA_SPARSE;
  else if (path == D2DMOE_PATH_AUTO && norms_in == nullptr && !sh.gated && sh.expert_dim > 64 && packed != nullptr &&
           sh.n_tokens > 16 && mfma_sparse_falls_back_to_sweep(sh))
    path = D2DMOE_PATH_MFMA_DENSE;   // a low fraction from a real router: d2dmoe_experts' own rule would still try the plan
  // ... and when the router kernel of this call is the one that walks the 32-token segments of that path's plan, it
  // leaves the plan's per-segment counts in the workspace on its way
  bool plan_counts_ready = false;
  if (norms_in == nullptr) {
    int32_t *seg_counts = nullptr, *seg_pairs = nullptr;
    // (only the fused router kernel does that: the buffer must hold this layer's router section)
    const bool router_in_packed = packed != nullptr && (packed_desc->sections & D2DMOE_SECTION_ROUTER) != 0 &&
                                  packed_desc->router_width == sh.router_width && sh.n_tokens > 16;
    if (path == D2DMOE_PATH_MFMA_SPARSE && router_in_packed && mfma_sparse_supported(sh) && mfma_router_writes_plan_counts(sh) &&
        plan.total - plan.perm_off >= mfma_sparse_workspace_bytes(sh)) {
      mfma_sparse_plan_counts(sh, ws + plan.perm_off, &seg_counts, &seg_pairs);
      plan_counts_ready = true;
    }
    st = router_select_impl(shape, x, router_w1, router_w2, packed, packed_desc, thr_scale, norms_out, routing, counts,
                            workspace, workspace_bytes, stream, seg_counts, seg_pairs);
  } else {
    st = d2dmoe_select(norms_in, routing, counts, sh.n_tokens, sh.n_experts, sh.dtype, thr_scale, stream);
  }
  if (st != D2DMOE_OK) return st;
  return experts_impl(shape, x, routing, w1, b1, w2, w_up, last_bias, packed, packed_desc, out, path, ws + plan.perm_off,
                      plan.total - plan.perm_off, stream, plan_counts_ready);
}

int d2dmoe_forward_static(const d2dmoe_shape* shape, const void* x, const void* router_w1, const void* router_w2,
                          float thr_scale, const void* w1, const void* b1, const void* w2, const void* w_up,
                          const void* last_bias, const void* packed, const d2dmoe_packed_desc* packed_desc,
                          const void* norms_in, void* norms_out, void* routing, int32_t* counts, void* out, int32_t path,
                          void* stream) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  if (plan_workspace(*shape).total > (size_t)D2DMOE_STATIC_WORKSPACE_BYTES) return D2DMOE_E_STATIC_LIMIT;
  st = check_packed(*shape, packed, packed_desc, false);   // host-only checks first: nothing below touches a device before them
  if (st != D2DMOE_OK) return st;
  void* ws = nullptr;
  st = static_scratch(&ws);
  if (st != D2DMOE_OK) return st;
  // Every kernel behind d2dmoe_forward initialises what it reads of its workspace (counters, flags, partial sums) on the
  // stream before use, so the contents the previous call left in the array are never seen.
  return d2dmoe_forward(shape, x, router_w1, router_w2, thr_scale, w1, b1, w2, w_up, last_bias, packed, packed_desc, norms_in,
                        norms_out, routing, counts, out, path, ws, (size_t)D2DMOE_STATIC_WORKSPACE_BYTES, stream);
}

size_t d2dmoe_norms_packed_bytes(const d2dmoe_shape* shape) {
  if (check_shape(shape) != D2DMOE_OK) return 0;
  return mfma_norms_packed_bytes(*shape);
}

int d2dmoe_pack_norms(const d2dmoe_shape* shape, const void* w1, const void* b1, const void* w2, void* packed,
                      size_t packed_bytes, void* stream) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  if (!w1 || !w2 || !packed) return D2DMOE_E_NULL;
  if (!mfma_norms_supported(*shape)) return D2DMOE_E_UNSUPPORTED;
  if (packed_bytes < mfma_norms_packed_bytes(*shape) || !aligned16(packed)) return D2DMOE_E_WORKSPACE;
  return (int)launch_norms_pack(*shape, w1, b1, w2, packed, (hipStream_t)stream);
}

int d2dmoe_expert_output_norms(const d2dmoe_shape* shape, const void* x, const void* packed, void* norms, void* stream) {
  int st = check_shape(shape);
  if (st != D2DMOE_OK) return st;
  if (shape->n_tokens == 0) return D2DMOE_OK;
  if (!x || !packed || !norms) return D2DMOE_E_NULL;
  if (!mfma_norms_supported(*shape)) return D2DMOE_E_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(packed)) return D2DMOE_E_ALIGN;
  return (int)launch_mfma_norms(*shape, x, packed, norms, (hipStream_t)stream);
}

}  // extern "C"
