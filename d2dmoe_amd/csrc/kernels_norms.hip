// L2 norm of every expert's output for every token -- the regression targets of router training -- without forming
// the outputs.  The reference runs the layer in 'masked' mode, captures the [E, N, D] expert outputs with a forward
// hook and takes vector_norm(ord=2, dim=-1) (moe_layers.py:125-133, 193-198; utils.py:353-369;
// train_routers.py:49-86).  Here, for expert e and token n with hidden activations h = act(x W1_e + b1_e):
//
//     |h W2_e|^2 = h (W2_e W2_e^T) h^T = h G_e h^T,        G_e: the expert's Ed x Ed Gram matrix, fixed per layer
//
// so the second layer shrinks from Ed x D to Ed x Ed per (token, expert) and the kernel is the first product of the
// dense sweep plus a 32 x 32 quadratic form.  bf16 inputs, float32 accumulation, h rounded to bf16 as the reference's
// tensors are; G enters as a bf16 pair (high part + remainder), which keeps it to float32-like accuracy.
//
// Layout: experts padded to 32 neurons, so a chunk of 256 neurons is 8 whole experts and wave w of the 4 owns experts
// 8 c + 2 w and 8 c + 2 w + 1 of chunk c.  A workgroup owns 64 tokens (x tile resident in LDS as B fragments, 96 KB).
//   GEMM1   H^T[64 neurons of the wave, 64 tokens] = W1^T . X^T   (v_mfma_f32_32x32x16_bf16, weight ring as in the
//           dense sweep); a lane ends with ONE token and 16 neurons per accumulator tile
//   h       + b1, activation, round to bf16: the registers are, as they stand, B fragments with K = the expert's
//           neurons in the order nu(half, g, i) = 16 half + 8 (i / 4) + 4 g + (i % 4)
//   T^T     = G_e . H_e^T with G_e fragments packed in that K order (4 MFMAs per expert and token tile): T^T has the
//           layout of H^T again, so |.|^2 = sum over the lane's 16 rows of T^T * H^T, plus the other lane half
//   norm    sqrt, round to bf16, 32 consecutive tokens per store: norms[e][n]
// Nothing goes through LDS after the x tile; the waves of a workgroup never wait for each other again.
#include "mfma_common.hpp"

namespace d2dmoe {

constexpr int NK_TT = 2;          // 32-token tiles per workgroup
constexpr int NK_EPC = 8;         // experts per chunk
constexpr int NK_RING = 32;

struct NormsLayout {
  int n_chunks;                   // ceil(E / 8)
  size_t w_off, b_off, g_off, total;
};

static NormsLayout norms_layout(const d2dmoe_shape& sh) {
  NormsLayout L;
  L.n_chunks = (sh.n_experts + NK_EPC - 1) / NK_EPC;
  const int ks1 = sh.d_model / 16;
  size_t off = 0;
  // per wave: n_chunks * 2 ks1 fragments, plus one ring of padding the last refills run into
  L.w_off = off; off += (size_t)MD_WAVES * ((size_t)L.n_chunks * 2 * ks1 + NK_RING) * 64 * 16;
  L.b_off = off; off += (size_t)L.n_chunks * MD_HC * 2;                        // bias, bf16, padded neurons zero
  off = (off + 255) / 256 * 256;
  L.g_off = off; off += (size_t)L.n_chunks * NK_EPC * 4 * 64 * 16;             // [expert][hi/lo][half][lane][8]
  L.total = (off + 255) / 256 * 256;
  return L;
}

bool mfma_norms_supported(const d2dmoe_shape& sh) {
  return sh.dtype == D2DMOE_BF16 && !sh.gated && sh.d_model == 768 && sh.expert_dim <= 32 && sh.n_experts <= 1024;
}

size_t mfma_norms_packed_bytes(const d2dmoe_shape& sh) { return mfma_norms_supported(sh) ? norms_layout(sh).total : 0; }

__device__ __forceinline__ int gram_k_order(int half, int g, int i) { return 16 * half + 8 * (i / 4) + 4 * g + (i % 4); }

// One thread per 16-byte piece of the weight stream, per bias element, per piece of the Gram fragments.
__global__ void pack_norms_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ b1, const bf16_t* __restrict__ w2,
                                  bf16_t* __restrict__ dw, bf16_t* __restrict__ db, bf16_t* __restrict__ dg, int D, int E, int Ed,
                                  int n_chunks) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int ks1 = D / 16;
  const int64_t per_wave = (int64_t)n_chunks * 2 * ks1 + NK_RING;   // fragments
  const int64_t n_w = (int64_t)MD_WAVES * per_wave * 64;
  const int64_t n_b = (int64_t)n_chunks * MD_HC;
  const int64_t n_g = (int64_t)n_chunks * NK_EPC * 4 * 64;
  if (p < n_w) {
    const int lane = (int)(p % 64);
    int64_t f = (p / 64) % per_wave;
    const int w = (int)(p / 64 / per_wave);
    const int g = lane >> 5, m = lane & 31;
    const bool pad = f >= per_wave - NK_RING;
    const int rt = (int)(f % 2); f /= 2;
    const int ks = (int)(f % ks1);
    const int c = (int)(f / ks1);
    const int e = c * NK_EPC + 2 * w + rt;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 16 + 8 * g + i;
      dw[p * 8 + i] = (!pad && e < E && m < Ed) ? w1[((int64_t)e * D + d) * Ed + m] : (bf16_t)0;
    }
  } else if (p < n_w + n_b) {
    const int64_t q = p - n_w;
    const int e = (int)(q / 32), j = (int)(q % 32);
    db[q] = (b1 != nullptr && e < E && j < Ed) ? b1[(int64_t)e * Ed + j] : (bf16_t)0;
  } else if (p < n_w + n_b + n_g) {
    const int64_t q = p - n_w - n_b;
    const int lane = (int)(q % 64);
    const int half = (int)((q / 64) % 2);
    const int hl = (int)((q / 128) % 2);
    const int e = (int)(q / 256);
    const int g = lane >> 5, m = lane & 31;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = gram_k_order(half, g, i);
      float acc = 0.f;
      if (e < E && m < Ed && j < Ed) {
        const bf16_t* ra = w2 + ((int64_t)e * Ed + m) * D;
        const bf16_t* rb = w2 + ((int64_t)e * Ed + j) * D;
        for (int d = 0; d < D; ++d) acc += bf16_to_f32(ra[d]) * bf16_to_f32(rb[d]);
      }
      const bf16_t hi = f32_to_bf16(acc);
      dg[q * 8 + i] = hl == 0 ? hi : f32_to_bf16(acc - bf16_to_f32(hi));
    }
  }
}

hipError_t launch_norms_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, void* packed, hipStream_t s) {
  const NormsLayout L = norms_layout(sh);
  char* base = (char*)packed;
  const int ks1 = sh.d_model / 16;
  const int64_t n = (int64_t)MD_WAVES * ((int64_t)L.n_chunks * 2 * ks1 + NK_RING) * 64 + (int64_t)L.n_chunks * MD_HC +
                    (int64_t)L.n_chunks * NK_EPC * 4 * 64;
  hipLaunchKernelGGL(pack_norms_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)w1, (const bf16_t*)b1,
                     (const bf16_t*)w2, (bf16_t*)(base + L.w_off), (bf16_t*)(base + L.b_off), (bf16_t*)(base + L.g_off),
                     sh.d_model, sh.n_experts, sh.expert_dim, L.n_chunks);
  return hipGetLastError();
}

struct NormsArgs {
  const bf16_t* x; const bf16x8* wp; const bf16_t* bias; const bf16x8* gram; bf16_t* norms;
  int64_t N; int E; int n_chunks; int act_rt;
  int n_full; int csplit; int chunks_per_split;   // workgroups [0, n_full) take whole tiles; the tiles after them are
                                                   // dealt to csplit workgroups each by chunk ranges (experts are
                                                   // independent, so nothing has to be summed afterwards)
};

template <int D, int ACT>
__global__ __launch_bounds__(256, 1) void expert_norms_kernel(const NormsArgs A) {
  constexpr int KS1 = D / 16;
  constexpr int TT = NK_TT;
  constexpr int BM = 32 * TT;
  constexpr int R = NK_RING;
  constexpr int NW1 = 2 * KS1;   // fragments per (wave, chunk)
  static_assert(NW1 % R == 0, "every chunk must start at ring slot 0");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16x8* xs = (bf16x8*)smem_raw;   // [TT][KS1][64]
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int g = lane >> 5, c32 = lane & 31;
  const int64_t N = A.N;
  const int n_chunks = A.n_chunks;
  int tile = (int)blockIdx.x, c_begin = 0, c_end = n_chunks;
  if (tile >= A.n_full) {
    const int idx = tile - A.n_full;
    tile = A.n_full + idx / A.csplit;
    c_begin = (idx % A.csplit) * A.chunks_per_split;
    c_end = (c_begin + A.chunks_per_split < n_chunks) ? (c_begin + A.chunks_per_split) : n_chunks;
  }
  const int64_t tok0 = (int64_t)tile * BM;

  // the weight stream of this wave: chunk-major, NW1 fragments per chunk, R fragments of padding at the end
  const bf16x8* wbase = A.wp + (int64_t)w * ((int64_t)n_chunks * NW1 + R) * 64 + lane;
  bf16x8 ring[R];
  // ---- x tile -> LDS as B fragments: lane (r, c) = (lane & 7, lane >> 3) takes row r of a block of 8 rows and the
  // 16-byte pieces c, c + 8, ...; rows past the end of the batch repeat the last row (their norms are not stored)
  {
    constexpr int RW = BM / 4, RB = RW / 8, XK = D / 64;
    const int r8 = lane & 7, c8l = lane >> 3;
    const int last_row = (int)((N - 1 - tok0) < (int64_t)(BM - 1) ? (N - 1 - tok0) : (int64_t)(BM - 1));
    u32x4 xv[RB][XK];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = w * RW + rb * 8 + r8;
      const u32x4* xrow = (const u32x4*)(A.x + (tok0 + (m < last_row ? m : last_row)) * D) + c8l;
#pragma unroll
      for (int kb = 0; kb < XK; ++kb) xv[rb][kb] = xrow[kb * 8];
    }
#pragma unroll
    for (int i = 0; i < R; ++i) ring[i] = wbase[((int64_t)c_begin * NW1 + i) * 64];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = w * RW + rb * 8 + r8;
      u32x4* xdst = (u32x4*)xs + ((m >> 5) * KS1 + (c8l >> 1)) * 64 + (m & 31) + 32 * (c8l & 1);
#pragma unroll
      for (int kb = 0; kb < XK; ++kb) xdst[kb * 4 * 64] = xv[rb][kb];
    }
  }
  lds_barrier();

  for (int c = c_begin; c < c_end; ++c) {
    const bf16x8* cur = wbase + (int64_t)c * NW1 * 64;
    const int e0 = c * NK_EPC + 2 * w;   // this wave's two experts of the chunk
    // Gram fragments and bias of the two experts: requested before the product, used after it
    bf16x8 gf[2][4];   // [expert][hi/lo * 2 + half]
    uint2 bq[2][4];    // [expert][accumulator quad]: 4 bf16 biases
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
      for (int k = 0; k < 4; ++k) gf[rt][k] = A.gram[((int64_t)(e0 + rt) * 4 + k) * 64 + lane];
#pragma unroll
      for (int q = 0; q < 4; ++q) bq[rt][q] = *(const uint2*)(A.bias + (int64_t)(e0 + rt) * 32 + 8 * q + 4 * g);
    }
    // ---- GEMM1
    f32x16 acc1[2][TT];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < TT; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc1[a][b][r] = 0.f;
    bf16x8 xb[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) xb[tt] = xs[tt * KS1 * 64 + lane];
    static_for<0, KS1>([&](auto ks_c) __attribute__((always_inline)) {
      constexpr int ks = decltype(ks_c)::value;
      const bf16x8 a0 = ring[(2 * ks) % R];
      const bf16x8 a1 = ring[(2 * ks + 1) % R];
      ring[(2 * ks) % R] = cur[(2 * ks + R) * 64];           // runs on into the next chunk (or the padding)
      ring[(2 * ks + 1) % R] = cur[(2 * ks + 1 + R) * 64];
      constexpr int kn = (ks + 1 < KS1) ? ks + 1 : ks;
      bf16x8 nxb[TT];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) nxb[tt] = xs[(tt * KS1 + kn) * 64 + lane];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        acc1[0][tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, xb[tt], acc1[0][tt], 0, 0, 0);
        acc1[1][tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, xb[tt], acc1[1][tt], 0, 0, 0);
      }
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) xb[tt] = nxb[tt];
      __builtin_amdgcn_sched_barrier(0);
    });
    // ---- hidden activations, quadratic form, norm
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int e = e0 + rt;
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        float hv[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float bias[4] = {__uint_as_float(bq[rt][q].x << 16), __uint_as_float(bq[rt][q].x & 0xffff0000u),
                                 __uint_as_float(bq[rt][q].y << 16), __uint_as_float(bq[rt][q].y & 0xffff0000u)};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float v = acc1[rt][tt][q * 4 + i] + bias[i];
            hv[q * 4 + i] = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(A.act_rt, v);
          }
        }
        bf16x8 hb[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          u32x4 pk;
          pk.x = pack2_bf16(hv[half * 8 + 0], hv[half * 8 + 1]);
          pk.y = pack2_bf16(hv[half * 8 + 2], hv[half * 8 + 3]);
          pk.z = pack2_bf16(hv[half * 8 + 4], hv[half * 8 + 5]);
          pk.w = pack2_bf16(hv[half * 8 + 6], hv[half * 8 + 7]);
          __builtin_memcpy(&hb[half], &pk, 16);
          // the rounded values, as the second factor of the quadratic form
          hv[half * 8 + 0] = __uint_as_float(pk.x << 16); hv[half * 8 + 1] = __uint_as_float(pk.x & 0xffff0000u);
          hv[half * 8 + 2] = __uint_as_float(pk.y << 16); hv[half * 8 + 3] = __uint_as_float(pk.y & 0xffff0000u);
          hv[half * 8 + 4] = __uint_as_float(pk.z << 16); hv[half * 8 + 5] = __uint_as_float(pk.z & 0xffff0000u);
          hv[half * 8 + 6] = __uint_as_float(pk.w << 16); hv[half * 8 + 7] = __uint_as_float(pk.w & 0xffff0000u);
        }
        f32x16 tq;
#pragma unroll
        for (int r = 0; r < 16; ++r) tq[r] = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) tq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gf[rt][k], hb[k & 1], tq, 0, 0, 0);
        float q2 = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) q2 += tq[r] * hv[r];
        q2 += __shfl_xor(q2, 32, 64);
        const int64_t n = tok0 + tt * 32 + c32;
        if (g == 0 && n < N && e < A.E) A.norms[(int64_t)e * N + n] = f32_to_bf16(sqrtf(fmaxf(q2, 0.f)));
      }
    }
  }
}

template <int ACT>
static hipError_t launch_norms_act(NormsArgs A, hipStream_t s) {
  constexpr int D = 768;
  const size_t lds = (size_t)NK_TT * (D / 16) * 64 * 16;
  auto kern = expert_norms_kernel<D, ACT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  // Whole tiles fill whole rounds of one workgroup per CU; a last, at most half-full round is spread over the machine
  // by chunk ranges.
  const int cus = device_cu_count();
  const int64_t tiles = (A.N + 32 * NK_TT - 1) / (32 * NK_TT);
  const int64_t leftover = tiles % cus;
  A.n_full = (int)tiles; A.csplit = 1; A.chunks_per_split = A.n_chunks;
  if (leftover > 0 && leftover * 2 <= cus && A.n_chunks >= 2) {
    int cs = (int)(cus / leftover);
    if (cs > A.n_chunks) cs = A.n_chunks;
    A.chunks_per_split = (A.n_chunks + cs - 1) / cs;
    A.csplit = (A.n_chunks + A.chunks_per_split - 1) / A.chunks_per_split;
    A.n_full = (int)(tiles - leftover);
  }
  const int64_t grid = A.n_full + (tiles - A.n_full) * A.csplit;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, s, A);
  return hipGetLastError();
}

hipError_t launch_mfma_norms(const d2dmoe_shape& sh, const void* x, const void* packed, void* norms, hipStream_t s) {
  const NormsLayout L = norms_layout(sh);
  const char* base = (const char*)packed;
  NormsArgs A;
  A.x = (const bf16_t*)x; A.wp = (const bf16x8*)(base + L.w_off); A.bias = (const bf16_t*)(base + L.b_off);
  A.gram = (const bf16x8*)(base + L.g_off); A.norms = (bf16_t*)norms;
  A.N = sh.n_tokens; A.E = sh.n_experts; A.n_chunks = L.n_chunks; A.act_rt = sh.activation;
  switch (sh.activation) {
    case D2DMOE_ACT_RELU: return launch_norms_act<D2DMOE_ACT_RELU>(A, s);
    case D2DMOE_ACT_GELU: return launch_norms_act<D2DMOE_ACT_GELU>(A, s);
    default: return launch_norms_act<-1>(A, s);
  }
}

}  // namespace d2dmoe
