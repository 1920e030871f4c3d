/*
 * d2dmoe.h -- C ABI of the MI355X (gfx950) dynamic-k MoE-FFN forward path.
 *
 * Every entry point
 *   - takes plain device pointers and sizes (no framework types),
 *   - enqueues its kernels on the HIP stream passed as `stream` (a hipStream_t cast to void*; NULL = the
 *     default stream) and returns without synchronising: no hipDeviceSynchronize, no device->host copies,
 *     no data-dependent launch shapes,
 *   - allocates and frees no device memory: outputs and the workspace belong to the caller,
 *   - returns D2DMOE_OK (0), a negative D2DMOE_E_* code for a rejected argument, or a positive hipError_t.
 *
 * "Reference" below is the D2DMoE repository; paths are relative to its root.
 *
 * Tensor layouts (row-major, contiguous; T = element type selected by `dtype`):
 *   x          [N, D]      T   tokens (the layer input flattened over batch and sequence)
 *   router_w1  [W, D]      T   first router Linear weight, [out, in] as nn.Linear stores it
 *   router_w2  [E, W]      T   second router Linear weight
 *   norms      [N, E]      T   predicted expert norms = router output
 *   routing    [N, E]      T   routing tensor; the gate writes exactly 0 or 1
 *   w1         [E, D, Ed]  T   expert up-projections        (gated experts: the gate projection)
 *   b1         [E, Ed]     T   expert first-layer biases, or NULL
 *   w2         [E, Ed, D]  T   expert down-projections
 *   w_up       [E, D, Ed]  T   gated experts only: the up projection, else NULL
 *   last_bias  [D]         T   output bias, or NULL
 *   out        [N, D]      T
 */
#ifndef D2DMOE_H
#define D2DMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define D2DMOE_VERSION 211 /* major*10000 + minor*100 + patch */

/* status codes */
enum {
  D2DMOE_OK = 0,
  D2DMOE_E_NULL = -1,        /* a required pointer is NULL */
  D2DMOE_E_SHAPE = -2,       /* a size is non-positive or outside what the kernels support */
  D2DMOE_E_DTYPE = -3,       /* unknown element type */
  D2DMOE_E_ACTIVATION = -4,  /* unknown activation */
  D2DMOE_E_WORKSPACE = -5,   /* workspace missing, misaligned or smaller than d2dmoe_workspace_bytes() */
  D2DMOE_E_UNSUPPORTED = -6, /* valid request that this build has no kernel for */
  D2DMOE_E_ALIGN = -7,       /* a tensor pointer is not aligned to 16 bytes */
  D2DMOE_E_STATIC_LIMIT = -8, /* d2dmoe_forward_static: the shape needs more than D2DMOE_STATIC_WORKSPACE_BYTES of workspace */
  D2DMOE_E_PACKED = -9       /* a packed buffer came without its descriptor, or the descriptor says it was packed for another
                                layer (shape, element type, sections) or by another layout version */
};

/* element types */
enum { D2DMOE_F32 = 0, D2DMOE_BF16 = 1, D2DMOE_F16 = 2 };   /* F16: every kernel family but the opt-in compacted one */

/* activations.  Reference: utils.py:730-756 (kernel-side definitions), common.py:159-169 (names). */
enum {
  D2DMOE_ACT_RELU = 0,       /* x >= 0 ? x : 0 */
  D2DMOE_ACT_GELU = 1,       /* erf form: x * 0.5 * (1 + erf(x / sqrt 2)) */
  D2DMOE_ACT_TANH = 2,
  D2DMOE_ACT_LEAKY_RELU = 3, /* slope 0.01 */
  D2DMOE_ACT_GELU_TANH = 4,  /* tanh approximation (stock Gemma) */
  D2DMOE_ACT_SILU = 5,
  D2DMOE_ACT_IDENTITY = 6,
  D2DMOE_ACT_ABS = 7
};

/* which expert kernel family d2dmoe_experts / d2dmoe_forward use */
enum {
  D2DMOE_PATH_AUTO = 0,       /* MFMA kernels when the shape and dtype have one, else the generic kernel */
  D2DMOE_PATH_GENERIC = 1,    /* token-tile-major scalar-FMA kernel: any shape, f32, bf16 or f16 storage, f32 math */
  D2DMOE_PATH_MFMA_DENSE = 2, /* bf16 or f16 MFMA, token-tile-major, masked dense sweep over all experts: ungated experts at
                                 D = 768 (hidden size up to 8192) or D = 1024 (up to 4096), at most 256 experts */
  D2DMOE_PATH_MFMA_SPARSE = 3, /* bf16 or f16 MFMA, expert-major over the permutation, then ordered combine; taken when at most
                                 8 experts per token are routed on average (checked on the device), else the dense sweep runs.  Ungated experts at D = 768 (also D = 1024 with at most 64 neurons and D = 1280 with at
                                 most 32: up to 12 / 6 experts per token; fall-back: the dense sweep at D = 1024, the tiled
                                 products at D = 1280 and wherever the sweep does not cover the layer).  Gated experts at D = 2048 with at most 64
                                 neurons: up to 32 experts per token (8 beyond 16 384 tokens), else the tiled products
                                 run.  d2dmoe_forward picks it under AUTO when thr_scale >= 0.75 (gated, or D other than 768: >= 0.5); for ungated
                                 experts of more than 64 neurons AUTO picks it in d2dmoe_experts, and in d2dmoe_forward when norms_in is
                                 given or thr_scale >= 0.5 */
  D2DMOE_PATH_MFMA_DECODE = 4, /* bf16 or f16 MFMA for a handful of tokens: per pass of 16 tokens one workgroup per expert streams
                                 that expert's packed weights once (gated or ungated experts); at most 48 tokens (three
                                 passes).  AUTO picks it up to 16 tokens, for gated experts up to 48 */
  D2DMOE_PATH_MFMA_MID = 6,   /* bf16 MFMA, ungated experts of at most 31 neurons at D = 768, at most 256 experts: work follows
                                 the routed pairs.  An expert-stationary first product gathers each expert's routed tokens
                                 (16 at a time, straight into registers) and keeps 64 bytes of hidden activations per pair;
                                 an output-stationary second product adds every expert's contribution, in ascending expert
                                 order, to float32 token rows held in LDS.  Runs when at most 48 experts per token are
                                 routed on average (checked on the device), else the dense sweep does.  Never picked by
                                 AUTO: it is ahead of the other paths only between about 7 and 9 experts per token */
  D2DMOE_PATH_MFMA_GEMM = 5   /* bf16 or f32 MFMA, D a multiple of 256, gated or ungated experts: two tiled products over all
                                 experts with the routing value as a factor of the hidden activations, which stay in
                                 the workspace between them; AUTO picks it for more than 16 tokens when the dense sweep
                                 does not cover the shape */
};

/* Shape of one MoE-FFN layer.  Mirrors the constructor arguments of the reference layer
 * (architectures/moe/moefication.py:30-52) and router (:310-326). */
typedef struct d2dmoe_shape {
  int64_t n_tokens;     /* N = batch * sequence */
  int32_t d_model;      /* D */
  int32_t n_experts;    /* E */
  int32_t expert_dim;   /* Ed, neurons per expert */
  int32_t router_width; /* W */
  int32_t dtype;        /* D2DMOE_F32 | D2DMOE_BF16 | D2DMOE_F16 (activations, weights, routing all share it) */
  int32_t activation;   /* expert activation, D2DMOE_ACT_* */
  int32_t gated;        /* 0: out = act(x w1 + b1) w2 ; 1: out = (act(x w1) * (x w_up)) w2 */
  int32_t add_residual; /* 1: out += x  (moefication.py:98-99) */
  int32_t router_activation;        /* hidden activation of the router MLP (D2DMoE: D2DMOE_ACT_RELU) */
  int32_t router_output_activation; /* output activation of the router MLP (D2DMoE: D2DMOE_ACT_ABS) */
} d2dmoe_shape;

/* What a buffer written by d2dmoe_pack_weights was packed for.  The pack call fills one (and writes the same 64 bytes at the
 * start of the buffer); every call that takes `packed` takes the descriptor next to it and checks it on the host against
 * its own `shape` before anything is launched -- device memory is never read for this.  A caller that keeps packed
 * buffers keeps their descriptors with them (or copies the buffer's first 64 bytes back and hands them to
 * d2dmoe_packed_desc_from_header).  No counterpart in the reference, which has no derived buffers. */
#define D2DMOE_PACKED_MAGIC 0x4b50324du   /* "M2PK" */
#define D2DMOE_PACKED_LAYOUT_VERSION 4u
enum {                       /* bits of d2dmoe_packed_desc.sections */
  D2DMOE_SECTION_DENSE = 1, D2DMOE_SECTION_EXPERT_MAJOR = 2, D2DMOE_SECTION_SMALL_BATCH = 4,
  D2DMOE_SECTION_TILED = 8, D2DMOE_SECTION_COMPACTED = 16, D2DMOE_SECTION_ROUTER = 32
};
typedef struct d2dmoe_packed_desc {
  uint32_t magic;           /* D2DMOE_PACKED_MAGIC */
  uint32_t layout_version;  /* D2DMOE_PACKED_LAYOUT_VERSION of the library that packed it */
  int32_t dtype, d_model, n_experts, expert_dim, gated;
  int32_t router_width;     /* router width the buffer was packed with (0: no router section) */
  uint32_t sections;        /* D2DMOE_SECTION_* present */
  uint32_t reserved0;
  uint64_t bytes;           /* size of the whole buffer, header included */
  uint64_t reserved1[2];
} d2dmoe_packed_desc;       /* 64 bytes */

/* The descriptor d2dmoe_pack_weights writes for `shape` (host only, nothing is launched): lets a caller see sections and
 * size ahead of packing.  D2DMOE_E_UNSUPPORTED when the shape has no packed buffer. */
int d2dmoe_packed_describe(const d2dmoe_shape* shape, d2dmoe_packed_desc* desc);

/* The descriptor found in a host copy of a packed buffer's first 64 bytes; D2DMOE_E_PACKED when they do not hold one. */
int d2dmoe_packed_desc_from_header(const void* host_header_64_bytes, d2dmoe_packed_desc* desc);

/* Library version (D2DMOE_VERSION of the build). */
int d2dmoe_version(void);

/* Text for a status code returned by this library (negative codes) or by HIP (positive codes). */
const char* d2dmoe_status_string(int status);

/* Bytes of caller-owned device workspace that d2dmoe_forward / d2dmoe_experts / d2dmoe_build_permutation
 * need for `shape` (the maximum over the three).  The workspace must be 256-byte aligned.  Replaces the
 * reference's internal torch.empty/torch.zeros temporaries (moe_impls.py:15, 190, 311). */
size_t d2dmoe_workspace_bytes(const d2dmoe_shape* shape);

/* Router MLP: norms = out_act(act(x W1^T) W2^T), depth 2, no biases.
 * Replaces MoeficationRouter.forward (architectures/moe/moefication.py:328-330) for the D2DMoE setting
 * (depth=2, bias=False; scripts/d2dmoe_vit_wallclock.py:318-325 uses act=relu, out_act=abs).
 * Intermediate and output are rounded to T after each layer, as eager nn.Linear does.
 * workspace: at least N*W*sizeof(T) bytes. */
int d2dmoe_router(const void* x, const void* router_w1, const void* router_w2, void* norms,
                  int64_t n_tokens, int32_t d_model, int32_t router_width, int32_t n_experts,
                  int32_t dtype, int32_t activation, int32_t output_activation,
                  void* workspace, size_t workspace_bytes, void* stream);

/* Dynamic-k selection: routing[n,e] = norms[n,e] >= round_T(max_e norms[n,:] * thr_scale) ? 1 : 0.
 * Replaces the 'dynk_max' branch of MoeficationMoE.gate (architectures/moe/moefication.py:80-85);
 * thr_scale is (float)(1.0 - tau).  NaN in a row propagates into its maximum, so that row selects nothing;
 * an all-zero row selects everything -- both as the reference's tensor ops behave.
 * counts (optional, int32 [E]) receives the number of tokens routed to each expert (it is zeroed here). */
int d2dmoe_select(const void* norms, void* routing, int32_t* counts, int64_t n_tokens, int32_t n_experts,
                  int32_t dtype, float thr_scale, void* stream);

/* Router MLP followed by dynamic-k selection in one call: d2dmoe_router then d2dmoe_select, with the router fixed
 * to shape->router_activation / router_output_activation.  With `packed` (from d2dmoe_pack_weights, router section
 * present) and a router the fused MFMA kernel covers, both stages run as ONE kernel and neither the hidden
 * activations nor the norms touch HBM unless norms_out is given.  Replaces the 'dynk_max' branch of
 * MoeficationMoE.gate including its router call (architectures/moe/moefication.py:80-85 -> :328-330).
 *   norms_out optional [N,E]; routing required [N,E]; counts optional int32 [E]
 * workspace: d2dmoe_workspace_bytes(shape) (only read when the fused kernel does not apply). */
int d2dmoe_router_select(const d2dmoe_shape* shape, const void* x, const void* router_w1, const void* router_w2,
                         const void* packed, const d2dmoe_packed_desc* packed_desc, float thr_scale, void* norms_out,
                         void* routing, int32_t* counts, void* workspace, size_t workspace_bytes, void* stream);

/* Token -> expert permutation from a routing tensor (entry > 0 means routed).
 * Replaces CustomKernelExperts.extract_indices / extract_indices_atomic
 * (architectures/moe/moe_layers.py:213-224, 241-249).  The order is canonical and deterministic: within an
 * expert, tokens ascend (the stable order; the reference's unstable argsort only defines the prefix sets).
 *   offsets      int32 [E+1]   exclusive prefix sum of the per-expert counts (offsets[E] = number of pairs)
 *   token_idx    int32 [N*E]   capacity N*E; the first offsets[E] entries are written: expert-major,
 *                              token-ascending list of routed tokens
 *   sort_indices   int64 [N,E] optional: column e = routed tokens ascending, then the other tokens ascending
 *                              (== argsort(routing.int(), dim=0, descending=True, stable=True))
 *   unsort_indices int64 [N,E] optional: per-column inverse of sort_indices
 *   bincounts      int64 [E]   optional: per-expert counts
 * workspace: d2dmoe_workspace_bytes() of a shape with the same N and E. */
int d2dmoe_build_permutation(const void* routing, int64_t n_tokens, int32_t n_experts, int32_t dtype,
                             int32_t* offsets, int32_t* token_idx,
                             int64_t* sort_indices, int64_t* unsort_indices, int64_t* bincounts,
                             void* workspace, size_t workspace_bytes, void* stream);

/* Experts: out[n,:] = sum_e routing[n,e] * expert_e(x[n,:]) (+ last_bias) (+ x[n,:]), summed in ascending
 * expert order in float32 with one final rounding to T; entries with routing == 0 are skipped.
 * Replaces CustomKernelExperts.forward in its 'triton'/'triton_atomic' modes
 * (architectures/moe/moe_layers.py:226-264 -> moe_impls.py:8-51, 183-204, 304-363) and, with gated = 1,
 * ExecuteAllExperts.forward with intermediate gating (moe_layers.py:86-96); last_bias / residual are the
 * epilogue of MoeficationMoE.forward (moefication.py:96-99).
 * For 0/1 routing this equals the reference's naive and Triton modes; for weighted routing it equals its
 * 'masked' mode (forward_all, moe_layers.py:193-198).
 * packed: optional buffer written by d2dmoe_pack_weights for the same weights (required by the MFMA paths;
 * D2DMOE_PATH_AUTO without it uses the generic kernel), with its descriptor: a buffer packed for another shape, element
 * type or layout version is refused with D2DMOE_E_PACKED (a buffer packed WITH a router section serves calls whose shape
 * names no router: the router section is the last one).
 * workspace: d2dmoe_workspace_bytes() of the same shape, 256-byte aligned.  Required by the expert-major, small-batch
 * and tiled-products paths; the dense sweep uses it when given (with few tokens it deals every tile's work to several
 * workgroups through it) and runs without it otherwise. */
int d2dmoe_experts(const d2dmoe_shape* shape, const void* x, const void* routing,
                   const void* w1, const void* b1, const void* w2, const void* w_up,
                   const void* last_bias, const void* packed, const d2dmoe_packed_desc* packed_desc, void* out,
                   int32_t path, void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of the derived weight buffer for the MFMA kernels (0 when `shape` has no MFMA kernel).  The buffer has one
 * section per kernel family that covers the shape (16-bit storage, i.e. bf16 or f16 -- dense sweep: D = 768 or 1024, ungated;
 * expert-major: ungated at D = 768 / 1024 / 1280, gated at D = 2048; small batch: D a multiple of 256 -- and tiled
 * products: bf16, f16 or f32, D a multiple of 256) and a router
 * section (when shape.router_width > 0 and the fused router+selection kernel covers the router: bf16 or f16, ReLU/abs,
 * hidden width 128 or 256, D a multiple of 64, and a number of experts that is a multiple of 8, at most 256). */
size_t d2dmoe_packed_bytes(const d2dmoe_shape* shape);

/* Re-tiles expert and router weights into MFMA fragment order.  A derived, cacheable buffer: call once per
 * weight update, with the same `shape` fields (other than n_tokens) that later calls will carry.  router_w1 and
 * router_w2 are required when the shape has a router section.  desc_out (required) receives the buffer's descriptor.
 * No counterpart in the reference (its Triton kernels re-read the nn.Parameter layout on every call). */
int d2dmoe_pack_weights(const d2dmoe_shape* shape, const void* w1, const void* b1, const void* w2,
                        const void* w_up, const void* router_w1, const void* router_w2,
                        void* packed, size_t packed_bytes, d2dmoe_packed_desc* desc_out, void* stream);

/* Whole layer: router -> dynamic-k select -> experts -> epilogue.
 * Replaces MoeficationMoE.forward with forward_mode == 'dynk_max'
 * (architectures/moe/moefication.py:90-101 calling :80-85 and the experts container).
 *   norms_in   optional [N,E]: when given, the router is skipped and these predicted norms are used -- the
 *              role of MoeficationRouter(test_override_outputs_p=...) (moefication.py:331-338)
 *   norms_out  optional [N,E]: receives the router output
 *   routing    required [N,E]: the routing tensor the layer returns next to its output
 *   counts     optional int32 [E]: tokens per expert */
int d2dmoe_forward(const d2dmoe_shape* shape, const void* x,
                   const void* router_w1, const void* router_w2, float thr_scale,
                   const void* w1, const void* b1, const void* w2, const void* w_up, const void* last_bias,
                   const void* packed, const d2dmoe_packed_desc* packed_desc, const void* norms_in,
                   void* norms_out, void* routing, int32_t* counts, void* out, int32_t path,
                   void* workspace, size_t workspace_bytes, void* stream);

/* d2dmoe_forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the same layer, the same kernels and bit-identical results, with the workspace taken
 * from an array that is part of the library's device code instead of a caller-owned buffer.  No counterpart in the
 * reference.  The entry point calls no hipMalloc / hipFree and no allocating library routine; the caller still passes
 * every input and output.
 *   - Limit: shapes whose d2dmoe_workspace_bytes() exceeds D2DMOE_STATIC_WORKSPACE_BYTES (256 MiB) are rejected with
 *     D2DMOE_E_STATIC_LIMIT before anything is launched (the ViT-B / GPT-2 layer fits up to 20 808 tokens, the
 *     Gemma-shape layer up to 2 027).  Each GPU the library runs on holds one such array until the process ends -- the
 *     array is part of the loaded code object, so every process that loads the library pays for it on every GPU it
 *     uses, whether or not it calls this entry point; a deployment that never does can build the library with a
 *     small D2DMOE_STATIC_WORKSPACE_BYTES.
 *   - Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race.  The
 *     array keeps the previous call's contents; the kernels initialise what they read of it on the stream, as they do
 *     with a caller-owned workspace.
 *   - The first call on each device looks the array's device address up (hipGetSymbolAddress); make that call outside
 *     stream capture. */
#ifndef D2DMOE_STATIC_WORKSPACE_BYTES   /* a build may size the array otherwise: hipcc -DD2DMOE_STATIC_WORKSPACE_BYTES=... */
#define D2DMOE_STATIC_WORKSPACE_BYTES (256u << 20)
#endif
int d2dmoe_forward_static(const d2dmoe_shape* shape, const void* x,
                          const void* router_w1, const void* router_w2, float thr_scale,
                          const void* w1, const void* b1, const void* w2, const void* w_up, const void* last_bias,
                          const void* packed, const d2dmoe_packed_desc* packed_desc, const void* norms_in,
                          void* norms_out, void* routing, int32_t* counts, void* out, int32_t path, void* stream);

/* L2 norm of every expert's output for every token, norms[e,n] = | act(x[n,:] . w1[e] + b1[e]) . w2[e] |_2 ([E,N]):
 * the regression targets of router training.  Replaces running the layer in 'masked' mode with a forward hook on
 * output_activation_extraction_stub that takes torch.linalg.vector_norm(output, ord=2, dim=-1) of the [E,N,D] expert
 * outputs (architectures/moe/moe_layers.py:125-133, 193-198; utils.py:353-369;
 * methods/dynamic_sparsification/train_routers.py:49-86).  The outputs are never formed: the second layer enters as
 * each expert's Ed x Ed Gram matrix.  bf16 or float16 (norms in the same type), D a multiple of 256 up to 2048, ungated
 * experts of at most 64 neurons, any activation; D2DMOE_E_UNSUPPORTED otherwise (d2dmoe_norms_packed_bytes then
 * returns 0).
 *   packed: d2dmoe_norms_packed_bytes(shape) bytes written by d2dmoe_pack_norms for the same weights (a derived,
 *           cacheable buffer of its own, separate from d2dmoe_pack_weights'); no workspace. */
size_t d2dmoe_norms_packed_bytes(const d2dmoe_shape* shape);
int d2dmoe_pack_norms(const d2dmoe_shape* shape, const void* w1, const void* b1, const void* w2,
                      void* packed, size_t packed_bytes, void* stream);
int d2dmoe_expert_output_norms(const d2dmoe_shape* shape, const void* x, const void* packed, void* norms,
                               void* stream);

#ifdef __cplusplus
}
#endif
#endif /* D2DMOE_H */
