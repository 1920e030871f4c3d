// L2 norm of every expert's output for every token -- the regression targets of router training -- without forming
// the outputs.  The reference runs the layer in 'masked' mode, captures the [E, N, D] expert outputs with a forward
// hook and takes vector_norm(ord=2, dim=-1) (moe_layers.py:125-133, 193-198; utils.py:353-369;
// train_routers.py:49-86).  Here, for expert e and token n with hidden activations h = act(x W1_e + b1_e):
//
//     |h W2_e|^2 = h (W2_e W2_e^T) h^T = h G_e h^T,        G_e: the expert's Ed x Ed Gram matrix, fixed per layer
//
// so the second layer shrinks from Ed x D to Ed x Ed per (token, expert) and the kernel is the first product of the
// dense sweep plus a quadratic form.  bf16 or float16 inputs, float32 accumulation, h rounded to the storage type as the
// reference's tensors are; G enters as a pair of 16-bit values (high part + remainder), which keeps it to float32-like
// accuracy.  In float16 an expert's G is scaled by a power of two so that its largest entry (a diagonal one) lies in
// [256, 512): entries stay clear of both ends of the float16 range whatever the weights' magnitude; the quadratic
// form is scaled back in float32.
//
// Layout: a chunk is 256 hidden rows = 8 slots of 32; wave w of the 4 owns slots 8 c + 2 w and 8 c + 2 w + 1 of chunk
// c.  Experts of at most 32 neurons take one slot each (padded to 32), experts of 33-64 neurons two (padded to 64; the
// wave's two slots are then one expert).  A workgroup owns 64 tokens (32 where D > 1024): x tile resident in LDS as B
// fragments, D / 8 KB per 32 tokens.  D is any multiple of 256 up to 2048 (the weight ring of 32 fragments then wraps
// at every chunk); D = 768 is compiled with the width as a constant.
//   GEMM1   H^T[64 rows of the wave, tokens] = W1^T . X^T   (v_mfma_f32_32x32x16_bf16 / _f16, weight ring as in the
//           dense sweep); a lane ends with ONE token and 16 neurons per accumulator tile
//   h       + b1, activation, round to the storage type: the registers are, as they stand, B fragments with K = the
//           slot's neurons in the order nu(half, g, i) = 16 half + 8 (i / 4) + 4 g + (i % 4)
//   T^T     = G . H^T with G's 32 x 32 blocks as fragments packed in that K order (4 MFMAs per block and token tile;
//           one block per small expert, 2 x 2 blocks per big one): T^T has the layout of H^T again, so
//           |.|^2 = sum over the lane's rows of T^T * H^T, plus the other lane half
//   norm    sqrt, round to the storage type, 32 consecutive tokens per store: norms[e][n]
// Nothing goes through LDS after the x tile; the waves of a workgroup never wait for each other again.
#include "mfma_common.hpp"

namespace d2dmoe {

constexpr int NK_SLOTS = 8;       // slots of 32 hidden rows per chunk
constexpr int NK_RING = 32;
constexpr int NK_MAX_D = 2048;

struct NormsLayout {
  bool wide;                      // experts of 33-64 neurons: two slots each
  int tt;                         // 32-token tiles per workgroup
  int n_chunks;                   // ceil(slots / 8)
  size_t w_off, b_off, g_off, s_off, total;
};

static NormsLayout norms_layout(const d2dmoe_shape& sh) {
  NormsLayout L;
  L.wide = sh.expert_dim > 32;
  L.tt = sh.d_model <= 1024 ? 2 : 1;
  const int slots = sh.n_experts * (L.wide ? 2 : 1);
  L.n_chunks = (slots + NK_SLOTS - 1) / NK_SLOTS;
  const int ks1 = sh.d_model / 16;
  size_t off = 0;
  // per wave: n_chunks * 2 ks1 fragments, plus one ring of padding the last refills run into
  L.w_off = off; off += (size_t)MD_WAVES * ((size_t)L.n_chunks * 2 * ks1 + NK_RING) * 64 * 16;
  L.b_off = off; off += (size_t)L.n_chunks * NK_SLOTS * 32 * 2;                 // bias, 16 bit, padded neurons zero
  off = (off + 255) / 256 * 256;
  // Gram fragments: [slot][hi/lo][half][lane][8], or [expert][row block][column block][hi/lo][half][lane][8]
  L.g_off = off; off += (size_t)L.n_chunks * NK_SLOTS * (L.wide ? 8 : 4) * 64 * 16;
  L.s_off = off; off += (size_t)L.n_chunks * NK_SLOTS * 4;                      // per slot: 1 / (power of two G was scaled by)
  L.total = (off + 255) / 256 * 256;
  return L;
}

bool mfma_norms_supported(const d2dmoe_shape& sh) {
  return (sh.dtype == D2DMOE_BF16 || sh.dtype == D2DMOE_F16) && !sh.gated && sh.d_model % 256 == 0 &&
         sh.d_model <= NK_MAX_D && sh.expert_dim <= 64 && sh.n_experts <= 1024;
}

size_t mfma_norms_packed_bytes(const d2dmoe_shape& sh) { return mfma_norms_supported(sh) ? norms_layout(sh).total : 0; }

__device__ __forceinline__ int gram_k_order(int half, int g, int i) { return 16 * half + 8 * (i / 4) + 4 * g + (i % 4); }

// One wave per expert: the power of two its Gram matrix is stored scaled by (float16 only; 1 in bf16), as its inverse.
// The largest entry of W2 W2^T is a diagonal one, the largest squared row norm of W2.
template <bool F16>
__global__ void norms_scale_kernel(const uint16_t* __restrict__ w2, float* __restrict__ inv_scale, int D, int E, int Ed, int wide,
                                   int n_slots) {
  const int e = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 6), lane = threadIdx.x & 63;
  if (e >= E) return;
  float inv = 1.f;
  if constexpr (F16) {
    float mx = 0.f;
    if (lane < Ed) {
      const uint16_t* row = w2 + ((int64_t)e * Ed + lane) * D;
      for (int d = 0; d < D; ++d) { const float v = dec16<F16>(row[d]); mx += v * v; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if (mx > 0.f && mx < 3.0e38f) inv = ldexpf(1.f, ilogbf(mx) - 8);
  }
  if (lane < (wide ? 2 : 1)) {
    const int slot = wide ? 2 * e + lane : e;
    if (slot < n_slots) inv_scale[slot] = inv;
  }
}

// One thread per 16-byte piece of the weight stream, per bias element, per piece of the Gram fragments.
template <bool F16>
__global__ void pack_norms_kernel(const uint16_t* __restrict__ w1, const uint16_t* __restrict__ b1, const uint16_t* __restrict__ w2,
                                  uint16_t* __restrict__ dw, uint16_t* __restrict__ db, uint16_t* __restrict__ dg,
                                  const float* __restrict__ inv_scale, int D, int E, int Ed, int n_chunks, int wide) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int ks1 = D / 16;
  const int64_t per_wave = (int64_t)n_chunks * 2 * ks1 + NK_RING;   // fragments
  const int64_t n_w = (int64_t)MD_WAVES * per_wave * 64;
  const int64_t n_b = (int64_t)n_chunks * NK_SLOTS * 32;
  const int64_t n_g = (int64_t)n_chunks * NK_SLOTS * (wide ? 8 : 4) * 64;
  if (p < n_w) {
    const int lane = (int)(p % 64);
    int64_t f = (p / 64) % per_wave;
    const int w = (int)(p / 64 / per_wave);
    const int g = lane >> 5, m = lane & 31;
    const bool pad = f >= per_wave - NK_RING;
    const int rt = (int)(f % 2); f /= 2;
    const int ks = (int)(f % ks1);
    const int c = (int)(f / ks1);
    const int slot = c * NK_SLOTS + 2 * w + rt;
    const int e = wide ? slot / 2 : slot;
    const int j = wide ? 32 * (slot % 2) + m : m;     // the expert's neuron
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = ks * 16 + 8 * g + i;
      dw[p * 8 + i] = (!pad && e < E && j < Ed) ? w1[((int64_t)e * D + d) * Ed + j] : (uint16_t)0;
    }
  } else if (p < n_w + n_b) {
    const int64_t q = p - n_w;
    const int slot = (int)(q / 32), m = (int)(q % 32);
    const int e = wide ? slot / 2 : slot;
    const int j = wide ? 32 * (slot % 2) + m : m;
    db[q] = (b1 != nullptr && e < E && j < Ed) ? b1[(int64_t)e * Ed + j] : (uint16_t)0;
  } else if (p < n_w + n_b + n_g) {
    const int64_t q = p - n_w - n_b;
    const int lane = (int)(q % 64);
    const int half = (int)((q / 64) % 2);
    const int hl = (int)((q / 128) % 2);
    int e, ra0, rb0;     // expert, first row / column of the 32 x 32 block
    if (wide) {
      const int cb = (int)((q / 256) % 2), rb = (int)((q / 512) % 2);
      e = (int)(q / 1024); ra0 = 32 * rb; rb0 = 32 * cb;
    } else {
      e = (int)(q / 256); ra0 = 0; rb0 = 0;
    }
    const int g = lane >> 5, m = ra0 + (lane & 31);
    const float sc = (e < E) ? 1.f / inv_scale[wide ? 2 * e : e] : 1.f;   // a power of two: exact
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = rb0 + gram_k_order(half, g, i);
      float acc = 0.f;
      if (e < E && m < Ed && j < Ed) {
        const uint16_t* ra = w2 + ((int64_t)e * Ed + m) * D;
        const uint16_t* rb = w2 + ((int64_t)e * Ed + j) * D;
        for (int d = 0; d < D; ++d) acc += dec16<F16>(ra[d]) * dec16<F16>(rb[d]);
      }
      acc *= sc;
      const uint16_t hi = enc16<F16>(acc);
      dg[q * 8 + i] = hl == 0 ? hi : enc16<F16>(acc - dec16<F16>(hi));
    }
  }
}

template <bool F16>
static hipError_t norms_pack_t(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, void* packed, hipStream_t s) {
  const NormsLayout L = norms_layout(sh);
  char* base = (char*)packed;
  const int ks1 = sh.d_model / 16;
  const int n_slots = L.n_chunks * NK_SLOTS;
  hipLaunchKernelGGL(norms_scale_kernel<F16>, dim3((unsigned)((sh.n_experts + 3) / 4)), dim3(256), 0, s, (const uint16_t*)w2,
                     (float*)(base + L.s_off), sh.d_model, sh.n_experts, sh.expert_dim, (int)L.wide, n_slots);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int64_t n = (int64_t)MD_WAVES * ((int64_t)L.n_chunks * 2 * ks1 + NK_RING) * 64 + (int64_t)n_slots * 32 +
                    (int64_t)n_slots * (L.wide ? 8 : 4) * 64;
  hipLaunchKernelGGL(pack_norms_kernel<F16>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const uint16_t*)w1,
                     (const uint16_t*)b1, (const uint16_t*)w2, (uint16_t*)(base + L.w_off), (uint16_t*)(base + L.b_off),
                     (uint16_t*)(base + L.g_off), (const float*)(base + L.s_off), sh.d_model, sh.n_experts, sh.expert_dim,
                     L.n_chunks, (int)L.wide);
  return hipGetLastError();
}

hipError_t launch_norms_pack(const d2dmoe_shape& sh, const void* w1, const void* b1, const void* w2, void* packed, hipStream_t s) {
  return sh.dtype == D2DMOE_F16 ? norms_pack_t<true>(sh, w1, b1, w2, packed, s) : norms_pack_t<false>(sh, w1, b1, w2, packed, s);
}

struct NormsArgs {
  const uint16_t* x; const bf16x8* wp; const uint16_t* bias; const bf16x8* gram; const float* inv_scale; uint16_t* norms;
  int64_t N; int D; int E; int n_chunks; int act_rt;
  int n_full; int csplit; int chunks_per_split;   // workgroups [0, n_full) take whole tiles; the tiles after them are
                                                   // dealt to csplit workgroups each by chunk ranges (experts are
                                                   // independent, so nothing has to be summed afterwards)
};

// DT: the width as a constant, or 0 for the width of the arguments (a multiple of 256).
template <int DT, int TT, bool F16, bool WIDE, int ACT>
__global__ __launch_bounds__(256, 1) void expert_norms_kernel(const NormsArgs A) {
  constexpr int BM = 32 * TT;
  constexpr int R = NK_RING;
  constexpr int KSB = R / 2;                 // K steps per turn of the ring
  const int D = DT ? DT : A.D;
  const int KS1 = D / 16;
  const int KB = KS1 / KSB;                  // turns of the ring per chunk (D / 256)
  const int NW1 = 2 * KS1;                   // fragments per (wave, chunk)
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
    constexpr int RW = BM / 4, RB = RW / 8;
    constexpr int XKMAX = (DT ? DT : (TT == 2 ? 1024 : NK_MAX_D)) / 64;   // pieces of 64 values a row can have
    const int XK = D / 64;
    const int r8 = lane & 7, c8l = lane >> 3;
    const int last_row = (int)((N - 1 - tok0) < (int64_t)(BM - 1) ? (N - 1 - tok0) : (int64_t)(BM - 1));
    u32x4 xv[RB][XKMAX];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = w * RW + rb * 8 + r8;
      const u32x4* xrow = (const u32x4*)(A.x + (tok0 + (m < last_row ? m : last_row)) * D) + c8l;
#pragma unroll
      for (int kb = 0; kb < XKMAX; kb += 4)
        if (kb < XK) {      // XK is a multiple of 4
#pragma unroll
          for (int k = kb; k < kb + 4; ++k) xv[rb][k] = xrow[k * 8];
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) ring[i] = wbase[((int64_t)c_begin * NW1 + i) * 64];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = w * RW + rb * 8 + r8;
      u32x4* xdst = (u32x4*)xs + ((m >> 5) * KS1 + (c8l >> 1)) * 64 + (m & 31) + 32 * (c8l & 1);
#pragma unroll
      for (int kb = 0; kb < XKMAX; kb += 4)
        if (kb < XK) {
#pragma unroll
          for (int k = kb; k < kb + 4; ++k) xdst[k * 4 * 64] = xv[rb][k];
        }
    }
  }
  lds_barrier();

  for (int c = c_begin; c < c_end; ++c) {
    const bf16x8* cur = wbase + (int64_t)c * NW1 * 64;
    const int s0 = c * NK_SLOTS + 2 * w;   // this wave's two slots of the chunk
    // Gram fragments, scale and bias of the two slots: requested before the product, used after it
    constexpr int NG = WIDE ? 16 : 8;
    bf16x8 gf[NG];     // narrow: [slot][hi/lo * 2 + half]; wide: [row block][column block][hi/lo * 2 + half]
    uint2 bq[2][4];    // [slot][accumulator quad]: 4 biases
    float inv[2];
#pragma unroll
    for (int k = 0; k < NG; ++k) gf[k] = A.gram[((int64_t)s0 * 4 * (WIDE ? 2 : 1) + k) * 64 + lane];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      inv[rt] = A.inv_scale[s0 + rt];
#pragma unroll
      for (int q = 0; q < 4; ++q) bq[rt][q] = *(const uint2*)(A.bias + (int64_t)(s0 + rt) * 32 + 8 * q + 4 * g);
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
    auto turn = [&](const int kb) __attribute__((always_inline)) {
      const bf16x8* curb = cur + (int64_t)kb * R * 64;
      const bf16x8* xsb = xs + kb * KSB * 64 + lane;
      static_for<0, KSB>([&](auto ks_c) __attribute__((always_inline)) {
        constexpr int ks = decltype(ks_c)::value;
        const bf16x8 a0 = ring[2 * ks];
        const bf16x8 a1 = ring[2 * ks + 1];
        ring[2 * ks] = curb[(2 * ks + R) * 64];           // runs on into the next chunk (or the padding)
        ring[2 * ks + 1] = curb[(2 * ks + 1 + R) * 64];
        const int kn = (kb * KSB + ks + 1 < KS1) ? ks + 1 : ks;
        bf16x8 nxb[TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) nxb[tt] = xsb[(tt * KS1 + kn) * 64];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          acc1[0][tt] = mfma_32x32x16<F16>(a0, xb[tt], acc1[0][tt]);
          acc1[1][tt] = mfma_32x32x16<F16>(a1, xb[tt], acc1[1][tt]);
        }
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) xb[tt] = nxb[tt];
        __builtin_amdgcn_sched_barrier(0);
      });
    };
    if constexpr (DT != 0) {
      static_for<0, DT / 16 / KSB>([&](auto kb_c) __attribute__((always_inline)) { turn(decltype(kb_c)::value); });
    } else {
      for (int kb = 0; kb < KB; ++kb) turn(kb);
    }
    // ---- hidden activations, quadratic form, norm
    float hv[2][TT][16];
    bf16x8 hb[2][TT][2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float bias[4] = {dec16<F16>(bq[rt][q].x & 0xffffu), dec16_hi<F16>(bq[rt][q].x),
                                 dec16<F16>(bq[rt][q].y & 0xffffu), dec16_hi<F16>(bq[rt][q].y)};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float v = acc1[rt][tt][q * 4 + i] + bias[i];
            hv[rt][tt][q * 4 + i] = (ACT >= 0) ? act_fn<ACT>(v) : apply_act(A.act_rt, v);
          }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          uint32_t pk[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            pk[k] = enc16x2<F16>(hv[rt][tt][half * 8 + 2 * k], hv[rt][tt][half * 8 + 2 * k + 1]);
            // the rounded values, as the second factor of the quadratic form
            hv[rt][tt][half * 8 + 2 * k] = dec16<F16>(pk[k] & 0xffffu);
            hv[rt][tt][half * 8 + 2 * k + 1] = dec16_hi<F16>(pk[k]);
          }
          const u32x4 pv = {pk[0], pk[1], pk[2], pk[3]};
          __builtin_memcpy(&hb[rt][tt][half], &pv, 16);
        }
      }
    }
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      float q2[2];
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {     // narrow: the slot's expert; wide: row block rt of the wave's one expert
        f32x16 tq;
#pragma unroll
        for (int r = 0; r < 16; ++r) tq[r] = 0.f;
        if constexpr (WIDE) {
#pragma unroll
          for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int k = 0; k < 4; ++k) tq = mfma_32x32x16<F16>(gf[(rt * 2 + cb) * 4 + k], hb[cb][tt][k & 1], tq);
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k) tq = mfma_32x32x16<F16>(gf[rt * 4 + k], hb[rt][tt][k & 1], tq);
        }
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += tq[r] * hv[rt][tt][r];
        q2[rt] = sum;
      }
      const int64_t n = tok0 + tt * 32 + c32;
      if constexpr (WIDE) {
        float q = q2[0] + q2[1];
        q += __shfl_xor(q, 32, 64);
        const int e = s0 / 2;
        if (g == 0 && n < N && e < A.E) A.norms[(int64_t)e * N + n] = enc16<F16>(sqrtf(fmaxf(q * inv[0], 0.f)));
      } else {
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
          float q = q2[rt];
          q += __shfl_xor(q, 32, 64);
          const int e = s0 + rt;
          if (g == 0 && n < N && e < A.E) A.norms[(int64_t)e * N + n] = enc16<F16>(sqrtf(fmaxf(q * inv[rt], 0.f)));
        }
      }
    }
  }
}

template <int DT, int TT, bool F16, bool WIDE, int ACT>
static hipError_t launch_norms_kernel(NormsArgs A, hipStream_t s) {
  const size_t lds = (size_t)TT * (A.D / 16) * 64 * 16;
  auto kern = expert_norms_kernel<DT, TT, F16, WIDE, ACT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  // Whole tiles fill whole rounds of one workgroup per CU; a last, at most half-full round is spread over the machine
  // by chunk ranges.
  const int cus = device_cu_count();
  const int64_t tiles = (A.N + 32 * TT - 1) / (32 * TT);
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

// The ViT-B / GPT-2-small / BERT-base case (D = 768, experts of at most 32 neurons) with width and activation compiled
// in; every other covered shape on the kernels that read both from the arguments.
template <bool F16>
static hipError_t launch_norms_t(const d2dmoe_shape& sh, const NormsLayout& L, const NormsArgs& A, hipStream_t s) {
  if (sh.d_model == 768 && !L.wide) {
    switch (sh.activation) {
      case D2DMOE_ACT_RELU: return launch_norms_kernel<768, 2, F16, false, D2DMOE_ACT_RELU>(A, s);
      case D2DMOE_ACT_GELU: return launch_norms_kernel<768, 2, F16, false, D2DMOE_ACT_GELU>(A, s);
      default: return launch_norms_kernel<768, 2, F16, false, -1>(A, s);
    }
  }
  if (L.tt == 2) return L.wide ? launch_norms_kernel<0, 2, F16, true, -1>(A, s) : launch_norms_kernel<0, 2, F16, false, -1>(A, s);
  return L.wide ? launch_norms_kernel<0, 1, F16, true, -1>(A, s) : launch_norms_kernel<0, 1, F16, false, -1>(A, s);
}

hipError_t launch_mfma_norms(const d2dmoe_shape& sh, const void* x, const void* packed, void* norms, hipStream_t s) {
  const NormsLayout L = norms_layout(sh);
  const char* base = (const char*)packed;
  NormsArgs A;
  A.x = (const uint16_t*)x; A.wp = (const bf16x8*)(base + L.w_off); A.bias = (const uint16_t*)(base + L.b_off);
  A.gram = (const bf16x8*)(base + L.g_off); A.inv_scale = (const float*)(base + L.s_off); A.norms = (uint16_t*)norms;
  A.N = sh.n_tokens; A.D = sh.d_model; A.E = sh.n_experts; A.n_chunks = L.n_chunks; A.act_rt = sh.activation;
  return sh.dtype == D2DMOE_F16 ? launch_norms_t<true>(sh, L, A, s) : launch_norms_t<false>(sh, L, A, s);
}

}  // namespace d2dmoe
