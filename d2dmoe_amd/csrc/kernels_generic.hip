// Generic (any-shape) kernels of the MoE-FFN forward path for gfx950: router linear layers, dynamic-k
// selection, token->expert permutation, and a token-tile-major experts kernel with float32 math.
// These are the float32 product path and the bf16 fallback for shapes without an MFMA kernel.
#include "common.hpp"
#include "launch.hpp"

namespace d2dmoe {

// =====================================================================================================
// Router layer:  C[M, Nout] = round_T(act(round_T(A[M,K] . B[Nout,K]^T)))
// (moefication.py:328-330: nn.Linear then the activation module, each producing a tensor of dtype T)
// 64x64 output tile per 256-thread workgroup, K staged through LDS in slabs of 16, 4x4 outputs per thread.
// =====================================================================================================
constexpr int LT_M = 64, LT_N = 64, LT_K = 16;

template <typename T>
__global__ __launch_bounds__(256) void linear_act_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                         T* __restrict__ C, int64_t M, int K, int Nout, int act) {
  __shared__ float As[LT_K][LT_M + 4];
  __shared__ float Bs[LT_K][LT_N + 4];
  const int t = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.x * LT_M;
  const int col0 = blockIdx.y * LT_N;
  const int lr = t >> 2;        // 0..63: tile row loaded by this thread
  const int lk = (t & 3) << 2;  // 0,4,8,12: first k of the 4 it loads
  const int ty = t >> 4, tx = t & 15;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += LT_K) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int64_t ar = row0 + lr;
      const int br = col0 + lr;
      As[lk + i][lr] = (ar < M && k < K) ? Elem<T>::load(A + ar * K + k) : 0.f;
      Bs[lk + i][lr] = (br < Nout && k < K) ? Elem<T>::load(B + (int64_t)br * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < LT_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t r = row0 + ty * 4 + i;
    if (r >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < Nout) {
        float v = Elem<T>::round(acc[i][j]);
        Elem<T>::store(C + r * Nout + c, apply_act(act, v));
      }
    }
  }
}

template <typename T>
hipError_t launch_linear_act(const void* A, const void* B, void* C, int64_t M, int K, int Nout, int act,
                             hipStream_t s) {
  dim3 grid((unsigned)cdiv64(M, LT_M), (unsigned)cdiv64(Nout, LT_N));
  hipLaunchKernelGGL(linear_act_kernel<T>, grid, dim3(256), 0, s, (const T*)A, (const T*)B, (T*)C, M, K, Nout, act);
  return hipGetLastError();
}
template hipError_t launch_linear_act<float>(const void*, const void*, void*, int64_t, int, int, int, hipStream_t);
template hipError_t launch_linear_act<bf16_t>(const void*, const void*, void*, int64_t, int, int, int, hipStream_t);
template hipError_t launch_linear_act<f16_t>(const void*, const void*, void*, int64_t, int, int, int, hipStream_t);

// The same layer in float32 on the matrix cores (v_mfma_f32_32x32x2_f32: float32 operands, products and sums), for
// K a multiple of 32 and Nout a multiple of 32.  Workgroup = 32 rows x 128 columns, one 32 x 32 tile per wave, no LDS:
// lane (c, h) holds 4 consecutive K values of row c of each operand per step of 8 (h = which half of the 8), read
// straight from global memory; the four waves share their A rows through the L1.  Two register buffers of 32 K values
// each alternate, so the loads of one are in flight while the other is multiplied.
typedef float f32x16_g __attribute__((ext_vector_type(16)));
typedef float f32x4_g __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void linear_act_mfma_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                                  float* __restrict__ C, int64_t M, int K, int Nout, int act) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int c32 = lane & 31, kh = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * 32;
  const int col0 = (blockIdx.y * 4 + w) * 32;
  if (col0 >= Nout) return;   // whole waves leave; the kernel has no barrier
  int64_t ar = row0 + c32;
  ar = ar < M ? ar : (M - 1);   // rows beyond M repeat the last row and are not stored
  const f32x4_g* ap = (const f32x4_g*)(A + ar * K) + kh;
  const f32x4_g* bp = (const f32x4_g*)(B + (int64_t)(col0 + c32) * K) + kh;
  f32x16_g acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  f32x4_g a0[4], b0[4], a1[4], b1[4];
  auto fill = [&](f32x4_g (&a)[4], f32x4_g (&b)[4], int k0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      a[u] = ap[(k0 >> 2) + 2 * u];
      b[u] = bp[(k0 >> 2) + 2 * u];
    }
  };
  auto multiply = [&](const f32x4_g (&a)[4], const f32x4_g (&b)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][q], b[u][q], acc, 0, 0, 0);
  };
  const int k_last = K - 32;
  fill(a0, b0, 0);
  for (int k0 = 0; k0 < K; k0 += 64) {
    fill(a1, b1, (k0 + 32 < K) ? (k0 + 32) : k_last);   // past the end: an in-bounds re-read that is not multiplied
    multiply(a0, b0);
    if (k0 + 32 < K) {
      fill(a0, b0, (k0 + 64 < K) ? (k0 + 64) : k_last);
      multiply(a1, b1);
    }
  }
  // lane = column c32; accumulator r = row 8*(r/4) + 4*kh + r%4
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int64_t row = row0 + 8 * (r / 4) + 4 * kh + (r % 4);
    if (row < M) C[row * Nout + col0 + c32] = apply_act(act, acc[r]);
  }
}

bool linear_mfma_f32_supported(int64_t M, int K, int Nout) { return M > 0 && K >= 32 && K % 32 == 0 && Nout % 32 == 0; }

hipError_t launch_linear_mfma_f32(const void* A, const void* B, void* C, int64_t M, int K, int Nout, int act, hipStream_t s) {
  dim3 grid((unsigned)cdiv64(M, 32), (unsigned)((Nout + 127) / 128));
  hipLaunchKernelGGL(linear_act_mfma_f32_kernel, grid, dim3(256), 0, s, (const float*)A, (const float*)B, (float*)C, M, K, Nout, act);
  return hipGetLastError();
}

// The same layer for float16 storage on the matrix cores (v_mfma_f32_32x32x16_f16: float32 sums), for K a multiple of
// 64 and Nout a multiple of 32; the arrangement of the float32 kernel above with 8 K values per lane and step of 16.
// The output is rounded to float16, then the activation is applied and rounded again, as the scalar kernel does.
typedef _Float16 f16x8_g __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(256) void linear_act_mfma_f16_kernel(const f16_t* __restrict__ A, const f16_t* __restrict__ B,
                                                                  f16_t* __restrict__ C, int64_t M, int K, int Nout, int act) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int c32 = lane & 31, kh = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * 32;
  const int col0 = (blockIdx.y * 4 + w) * 32;
  if (col0 >= Nout) return;   // whole waves leave; the kernel has no barrier
  int64_t ar = row0 + c32;
  ar = ar < M ? ar : (M - 1);   // rows beyond M repeat the last row and are not stored
  const f16x8_g* ap = (const f16x8_g*)(A + ar * K) + kh;
  const f16x8_g* bp = (const f16x8_g*)(B + (int64_t)(col0 + c32) * K) + kh;
  f32x16_g acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  f16x8_g a0[4], b0[4], a1[4], b1[4];   // two buffers of 64 K values
  auto fill = [&](f16x8_g (&a)[4], f16x8_g (&b)[4], int k0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      a[u] = ap[(k0 >> 3) + 2 * u];
      b[u] = bp[(k0 >> 3) + 2 * u];
    }
  };
  auto multiply = [&](const f16x8_g (&a)[4], const f16x8_g (&b)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[u], b[u], acc, 0, 0, 0);
  };
  const int k_last = K - 64;
  fill(a0, b0, 0);
  for (int k0 = 0; k0 < K; k0 += 128) {
    fill(a1, b1, (k0 + 64 < K) ? (k0 + 64) : k_last);   // past the end: an in-bounds re-read that is not multiplied
    multiply(a0, b0);
    if (k0 + 64 < K) {
      fill(a0, b0, (k0 + 128 < K) ? (k0 + 128) : k_last);
      multiply(a1, b1);
    }
  }
  // lane = column c32; accumulator r = row 8*(r/4) + 4*kh + r%4
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int64_t row = row0 + 8 * (r / 4) + 4 * kh + (r % 4);
    if (row < M) Elem<f16_t>::store(C + row * Nout + col0 + c32, apply_act(act, Elem<f16_t>::round(acc[r])));
  }
}

bool linear_mfma_f16_supported(int64_t M, int K, int Nout) { return M > 0 && K >= 64 && K % 64 == 0 && Nout % 32 == 0; }

hipError_t launch_linear_mfma_f16(const void* A, const void* B, void* C, int64_t M, int K, int Nout, int act, hipStream_t s) {
  dim3 grid((unsigned)cdiv64(M, 32), (unsigned)((Nout + 127) / 128));
  hipLaunchKernelGGL(linear_act_mfma_f16_kernel, grid, dim3(256), 0, s, (const f16_t*)A, (const f16_t*)B, (f16_t*)C, M, K, Nout, act);
  return hipGetLastError();
}

// =====================================================================================================
// small fill kernel (used instead of a memset node so the path stays graph-capture friendly)
// =====================================================================================================
__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}
hipError_t launch_fill_i32(int32_t* p, int64_t n, int32_t v, hipStream_t s) {
  int blocks = (int)(cdiv64(n, 256) < 1024 ? cdiv64(n, 256) : 1024);
  hipLaunchKernelGGL(fill_i32_kernel, dim3(blocks), dim3(256), 0, s, p, n, v);
  return hipGetLastError();
}

// =====================================================================================================
// Dynamic-k selection (moefication.py:80-85).  One wave per token row; lanes stride over the experts.
//   m   = max_e norms[n,e]            (NaN-propagating, as torch.max)
//   thr = round_T(float(m) * thr_scale)
//   routing[n,e] = norms[n,e] >= thr ? 1 : 0
// Optional per-expert token counts: accumulated per lane over the wave's rows, then one integer atomic per
// (wave, expert) -- integer adds, so the result does not depend on the order.
// =====================================================================================================
constexpr int SEL_MAX_VPT = 16;  // experts per lane -> E <= 1024

template <typename T>
__global__ __launch_bounds__(256) void select_kernel(const T* __restrict__ norms, T* __restrict__ routing,
                                                     int32_t* __restrict__ counts, int64_t N, int E,
                                                     float thr_scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  const int64_t n_waves = ((int64_t)gridDim.x * blockDim.x) / kWave;
  const int vpt = (E + kWave - 1) / kWave;
  int cnt[SEL_MAX_VPT];
#pragma unroll
  for (int k = 0; k < SEL_MAX_VPT; ++k) cnt[k] = 0;
  for (int64_t n = wave; n < N; n += n_waves) {
    float v[SEL_MAX_VPT];
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < SEL_MAX_VPT; ++k) {
      if (k < vpt) {
        const int e = lane + k * kWave;
        const float nv = Elem<T>::load(norms + n * E + (e < E ? e : E - 1));   // unconditional (clamped) load
        v[k] = (e < E) ? nv : -INFINITY;
        m = nanmax(m, v[k]);
      }
    }
    m = wave_nanmax(m);
    // the product is rounded to float32 first, then to T, as the reference's tensor expression does on a GPU; without the
    // empty asm the compiler folds multiply and conversion to float16 into one mixed-precision instruction with a
    // single rounding, which differs when the float32 product is an exact tie of the float16 grid
    float prod = m * thr_scale;
    asm volatile("" : "+v"(prod));
    const float thr = Elem<T>::round(prod);
#pragma unroll
    for (int k = 0; k < SEL_MAX_VPT; ++k) {
      if (k < vpt) {
        const int e = lane + k * kWave;
        if (e < E) {
          const bool on = v[k] >= thr;
          Elem<T>::store(routing + n * E + e, on ? 1.f : 0.f);
          cnt[k] += on ? 1 : 0;
        }
      }
    }
  }
  if (counts != nullptr) {
#pragma unroll
    for (int k = 0; k < SEL_MAX_VPT; ++k) {
      if (k < vpt) {
        const int e = lane + k * kWave;
        if (e < E && cnt[k] != 0) atomicAdd(counts + e, cnt[k]);
      }
    }
  }
}

template <typename T>
hipError_t launch_select(const void* norms, void* routing, int32_t* counts, int64_t N, int E, float thr_scale,
                         hipStream_t s) {
  if (counts != nullptr) {
    hipError_t e = launch_fill_i32(counts, E, 0, s);
    if (e != hipSuccess) return e;
  }
  int64_t blocks = cdiv64(N, 4);
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(select_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, (const T*)norms, (T*)routing, counts,
                     N, E, thr_scale);
  return hipGetLastError();
}
template hipError_t launch_select<float>(const void*, void*, int32_t*, int64_t, int, float, hipStream_t);
template hipError_t launch_select<bf16_t>(const void*, void*, int32_t*, int64_t, int, float, hipStream_t);
template hipError_t launch_select<f16_t>(const void*, void*, int32_t*, int64_t, int, float, hipStream_t);

// =====================================================================================================
// Token -> expert permutation (moe_layers.py:213-224, 241-249), canonical stable order.
// Tokens are cut into segments of 64.  Lanes map to experts, so every load of a routing row is coalesced and
// a per-lane running counter IS the rank of the current token inside its expert's list.
//   pass 1  perm_count_kernel   seg_counts[seg][e]
//   pass 2  perm_scan_kernel    seg_offsets[seg][e] = exclusive prefix over segments; totals[e]
//   pass 3  perm_offsets_kernel offsets[E+1] = exclusive prefix over experts (+ int64 bincounts)
//   pass 4  perm_scatter_kernel token_idx, optional sort_indices / unsort_indices
// =====================================================================================================
constexpr int PERM_SEG = 64;
constexpr int PERM_MAX_VPT = 16;  // E <= 1024

template <typename T>
__global__ __launch_bounds__(256) void perm_count_kernel(const T* __restrict__ routing, int32_t* __restrict__ seg_counts,
                                                         int64_t N, int E, int64_t n_seg) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t seg = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  if (seg >= n_seg) return;
  const int vpt = (E + kWave - 1) / kWave;
  const int64_t t0 = seg * PERM_SEG;
  const int rows = (int)((N - t0) < PERM_SEG ? (N - t0) : PERM_SEG);
  int cnt[PERM_MAX_VPT];
#pragma unroll
  for (int k = 0; k < PERM_MAX_VPT; ++k) cnt[k] = 0;
  // a lane group's whole segment is requested at once, every load unconditional (clamped address): one round trip
  // to memory per group of 64 experts
#pragma unroll
  for (int k = 0; k < PERM_MAX_VPT; ++k) {
    if (k < vpt) {
      const int e = lane + k * kWave;
      const int ec = (e < E) ? e : (E - 1);
      float v[PERM_SEG];
#pragma unroll
      for (int i = 0; i < PERM_SEG; ++i) {
        const int r = (i < rows) ? i : (rows - 1);
        v[i] = Elem<T>::load(routing + (t0 + r) * E + ec);
      }
#pragma unroll
      for (int i = 0; i < PERM_SEG; ++i) cnt[k] += (i < rows && e < E && v[i] > 0.f) ? 1 : 0;
    }
  }
#pragma unroll
  for (int k = 0; k < PERM_MAX_VPT; ++k) {
    if (k < vpt) {
      const int e = lane + k * kWave;
      if (e < E) seg_counts[seg * E + e] = cnt[k];
    }
  }
}

// Exclusive prefix over segments, per expert.  Grid = (groups of 64 experts) x (PERM_SCAN_BLOCKS blocks of consecutive
// segments); a workgroup has 16 waves, lanes = experts.  A workgroup first adds up everything before its block (its
// waves share that range), then wave w scans its own slice of the block; partial sums meet in LDS.  Integer sums, so
// the result does not depend on the split.
constexpr int PERM_SCAN_BLOCKS = 32;

__global__ __launch_bounds__(1024) void perm_scan_kernel(const int32_t* __restrict__ seg_counts,
                                                         int32_t* __restrict__ seg_offsets, int32_t* __restrict__ totals,
                                                         int E, int64_t n_seg) {
  __shared__ int32_t before[16][kWave];
  __shared__ int32_t part[16][kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x / kWave;
  const int e = blockIdx.x * kWave + lane;
  const int64_t per_block = (n_seg + PERM_SCAN_BLOCKS - 1) / PERM_SCAN_BLOCKS;
  const int64_t b0 = ((int64_t)blockIdx.y * per_block) < n_seg ? ((int64_t)blockIdx.y * per_block) : n_seg;
  const int64_t b1 = (b0 + per_block) < n_seg ? (b0 + per_block) : n_seg;
  // segments [0, b0) split over the waves
  const int64_t pa = (b0 + 15) / 16;
  const int64_t a0 = (w * pa) < b0 ? (w * pa) : b0;
  const int64_t a1 = (a0 + pa) < b0 ? (a0 + pa) : b0;
  // this wave's slice of [b0, b1)
  const int64_t per = (b1 > b0) ? ((b1 - b0 + 15) / 16) : 0;
  const int64_t s0 = (b0 + w * per) < b1 ? (b0 + w * per) : b1;
  const int64_t s1 = (s0 + per) < b1 ? (s0 + per) : b1;
  int pre = 0, sum = 0;
  if (e < E) {
#pragma unroll 16
    for (int64_t s = a0; s < a1; ++s) pre += seg_counts[s * E + e];
#pragma unroll 16
    for (int64_t s = s0; s < s1; ++s) sum += seg_counts[s * E + e];
  }
  before[w][lane] = pre;
  part[w][lane] = sum;
  __syncthreads();
  int run = 0;
  for (int i = 0; i < 16; ++i) run += before[i][lane];
  for (int i = 0; i < w; ++i) run += part[i][lane];
  if (e < E) {
#pragma unroll 16
    for (int64_t s = s0; s < s1; ++s) {
      const int c = seg_counts[s * E + e];
      seg_offsets[s * E + e] = run;
      run += c;
    }
    if (w == 15 && blockIdx.y == PERM_SCAN_BLOCKS - 1) totals[e] = run;
  }
}

// offsets[E+1] from totals[E]; single workgroup, E <= 1024.
__global__ __launch_bounds__(1024) void perm_offsets_kernel(const int32_t* __restrict__ totals, int32_t* __restrict__ offsets,
                                                            int64_t* __restrict__ bincounts, int E) {
  __shared__ int32_t buf[1024];
  const int t = threadIdx.x;
  const int c = (t < E) ? totals[t] : 0;
  buf[t] = c;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {  // Hillis-Steele inclusive scan
    int v = (t >= off) ? buf[t - off] : 0;
    __syncthreads();
    buf[t] += v;
    __syncthreads();
  }
  if (t < E) {
    offsets[t + 1] = buf[t];
    if (bincounts != nullptr) bincounts[t] = c;
  }
  if (t == 0) offsets[0] = 0;
}

template <typename T>
__global__ __launch_bounds__(256) void perm_scatter_kernel(const T* __restrict__ routing, const int32_t* __restrict__ seg_offsets,
                                                           const int32_t* __restrict__ offsets, int32_t* __restrict__ token_idx,
                                                           int64_t* __restrict__ sort_indices, int64_t* __restrict__ unsort_indices,
                                                           int64_t N, int E, int64_t n_seg) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t seg = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  if (seg >= n_seg) return;
  const int vpt = (E + kWave - 1) / kWave;
  const int64_t t0 = seg * PERM_SEG;
  const int rows = (int)((N - t0) < PERM_SEG ? (N - t0) : PERM_SEG);
  int run[PERM_MAX_VPT];   // routed tokens of expert e before the current token
  int base[PERM_MAX_VPT];  // offsets[e]
  int total[PERM_MAX_VPT]; // count[e]
#pragma unroll
  for (int k = 0; k < PERM_MAX_VPT; ++k) {
    run[k] = 0; base[k] = 0; total[k] = 0;
    if (k < vpt) {
      const int e = lane + k * kWave;
      if (e < E) {
        run[k] = seg_offsets[seg * E + e];
        base[k] = offsets[e];
        total[k] = offsets[e + 1] - offsets[e];
      }
    }
  }
  // the segment's routing entries of this lane's experts as bit masks (bit i = token i routes to the expert); a lane
  // group's rows are requested together, unconditionally (clamped addresses)
  static_assert(PERM_SEG <= 64, "one 64-bit mask per lane group");
  unsigned long long onbits[PERM_MAX_VPT];
#pragma unroll
  for (int k = 0; k < PERM_MAX_VPT; ++k) {
    onbits[k] = 0ull;
    if (k < vpt) {
      const int e = lane + k * kWave;
      const int ec = (e < E) ? e : (E - 1);
      float v[PERM_SEG];
#pragma unroll
      for (int i = 0; i < PERM_SEG; ++i) {
        const int r = (i < rows) ? i : (rows - 1);
        v[i] = Elem<T>::load(routing + (t0 + r) * E + ec);
      }
#pragma unroll
      for (int i = 0; i < PERM_SEG; ++i) onbits[k] |= (unsigned long long)(v[i] > 0.f ? 1 : 0) << i;
    }
  }
  if (sort_indices == nullptr && unsort_indices == nullptr) {
    // only the per-expert token lists are wanted: a lane walks the set bits of its experts' masks (the routed tokens, in
    // ascending order) instead of all the segment's tokens
#pragma unroll
    for (int k = 0; k < PERM_MAX_VPT; ++k) {
      if (k < vpt) {
        // (rows past the end of the batch and lanes past the last expert hold copies of clamped loads: masked here)
        const unsigned long long live = (rows >= 64) ? ~0ull : ((1ull << rows) - 1ull);
        unsigned long long bits = (lane + k * kWave < E) ? (onbits[k] & live) : 0ull;
        int64_t pos = (int64_t)base[k] + run[k];
        while (bits != 0ull) {
          token_idx[pos++] = (int32_t)(t0 + __builtin_ctzll(bits));
          bits &= bits - 1ull;
        }
      }
    }
    return;
  }
  for (int i = 0; i < rows; ++i) {
    const int64_t tok = t0 + i;
#pragma unroll
    for (int k = 0; k < PERM_MAX_VPT; ++k) {
      if (k < vpt) {
        const int e = lane + k * kWave;
        if (e < E) {
          const bool on = ((onbits[k] >> i) & 1ull) != 0ull;
          // position inside column e of the full (routed first, then the rest) ordering
          const int64_t pos = on ? (int64_t)run[k] : (int64_t)total[k] + (tok - run[k]);
          if (on) token_idx[(int64_t)base[k] + run[k]] = (int32_t)tok;
          if (sort_indices != nullptr) sort_indices[pos * E + e] = tok;
          if (unsort_indices != nullptr) unsort_indices[tok * E + e] = pos;
          run[k] += on ? 1 : 0;
        }
      }
    }
  }
}

void launch_perm_scan(const int32_t* seg_counts, int32_t* seg_offsets, int32_t* totals, int E, int64_t n_seg, hipStream_t s) {
  hipLaunchKernelGGL(perm_scan_kernel, dim3((E + kWave - 1) / kWave, PERM_SCAN_BLOCKS), dim3(1024), 0, s, seg_counts, seg_offsets, totals, E, n_seg);
}

size_t perm_workspace_bytes(int64_t N, int E) {
  const int64_t n_seg = cdiv64(N, PERM_SEG);
  // seg_counts + seg_offsets + totals
  return (size_t)(2 * n_seg * E + E) * sizeof(int32_t);
}

template <typename T>
hipError_t launch_build_permutation(const void* routing, int64_t N, int E, int32_t* offsets, int32_t* token_idx,
                                    int64_t* sort_indices, int64_t* unsort_indices, int64_t* bincounts,
                                    void* workspace, hipStream_t s) {
  const int64_t n_seg = cdiv64(N, PERM_SEG);
  int32_t* seg_counts = (int32_t*)workspace;
  int32_t* seg_offsets = seg_counts + n_seg * E;
  int32_t* totals = seg_offsets + n_seg * E;
  const unsigned seg_blocks = (unsigned)cdiv64(n_seg, 4);
  hipLaunchKernelGGL(perm_count_kernel<T>, dim3(seg_blocks), dim3(256), 0, s, (const T*)routing, seg_counts, N, E, n_seg);
  hipLaunchKernelGGL(perm_scan_kernel, dim3((E + kWave - 1) / kWave, PERM_SCAN_BLOCKS), dim3(1024), 0, s, seg_counts, seg_offsets, totals, E, n_seg);
  hipLaunchKernelGGL(perm_offsets_kernel, dim3(1), dim3(1024), 0, s, totals, offsets, bincounts, E);
  hipLaunchKernelGGL(perm_scatter_kernel<T>, dim3(seg_blocks), dim3(256), 0, s, (const T*)routing, seg_offsets, offsets,
                     token_idx, sort_indices, unsort_indices, N, E, n_seg);
  return hipGetLastError();
}
template hipError_t launch_build_permutation<float>(const void*, int64_t, int, int32_t*, int32_t*, int64_t*, int64_t*,
                                                    int64_t*, void*, hipStream_t);
template hipError_t launch_build_permutation<bf16_t>(const void*, int64_t, int, int32_t*, int32_t*, int64_t*, int64_t*,
                                                     int64_t*, void*, hipStream_t);
template hipError_t launch_build_permutation<f16_t>(const void*, int64_t, int, int32_t*, int32_t*, int64_t*, int64_t*,
                                                     int64_t*, void*, hipStream_t);

// =====================================================================================================
// Experts, generic token-tile-major kernel.
// A workgroup owns BM tokens: their rows of x and routing sit in LDS for the whole kernel, and the output tile
// [BM, D] lives in registers (thread t owns columns t, t+256, ...).  Experts are visited in ascending order;
// an expert that no token of the tile routes to is skipped (uniform branch).  For each visited expert:
//   h[m,j]   = round_T(act(x[m,:] . w1[e,:,j] + b1[e,j]))          (gated: act(x.w1) * (x.w_up))
//   acc[m,c] += (routing[m,e] * h[m,j]) * w2[e,j,c]
// so the sum over experts is taken in ascending expert order in float32 and rounded once at the end
// (the order of moe_merge_results_kernel, moe_impls.py:499-514).  Epilogue: + last_bias, + x (residual).
// =====================================================================================================
template <typename T, int BM, int CPT>
__global__ __launch_bounds__(256) void experts_generic_kernel(
    const T* __restrict__ x, const T* __restrict__ routing, const T* __restrict__ w1, const T* __restrict__ b1,
    const T* __restrict__ w2, const T* __restrict__ w_up, const T* __restrict__ last_bias, T* __restrict__ out,
    int64_t N, int D, int E, int Ed, int act, int add_residual) {
  extern __shared__ float smem[];
  float* xs = smem;                 // [BM][D]
  float* rs = xs + BM * D;          // [BM][E]
  float* hs = rs + BM * E;          // [BM][Ed]
  int* active = (int*)(hs + BM * Ed);  // [E]
  const int t = threadIdx.x;
  const int64_t tok0 = (int64_t)blockIdx.x * BM;

  for (int i = t; i < BM * D; i += 256) {
    const int m = i / D, d = i - m * D;
    const int64_t n = tok0 + m;
    xs[i] = (n < N) ? Elem<T>::load(x + n * D + d) : 0.f;
  }
  for (int i = t; i < BM * E; i += 256) {
    const int m = i / E, e = i - m * E;
    const int64_t n = tok0 + m;
    rs[i] = (n < N) ? Elem<T>::load(routing + n * E + e) : 0.f;
  }
  __syncthreads();
  for (int e = t; e < E; e += 256) {
    int any = 0;
    for (int m = 0; m < BM; ++m) any |= (rs[m * E + e] != 0.f) ? 1 : 0;
    active[e] = any;
  }
  __syncthreads();

  float acc[BM][CPT];
#pragma unroll
  for (int m = 0; m < BM; ++m)
#pragma unroll
    for (int c = 0; c < CPT; ++c) acc[m][c] = 0.f;

  for (int e = 0; e < E; ++e) {
    if (!active[e]) continue;
    const T* w1e = w1 + (int64_t)e * D * Ed;
    const T* wue = (w_up != nullptr) ? (w_up + (int64_t)e * D * Ed) : nullptr;
    for (int p = t; p < BM * Ed; p += 256) {
      const int m = p / Ed, j = p - m * Ed;
      const float* xr = xs + m * D;
      float a = 0.f, u = 0.f;
      if (wue == nullptr) {
        for (int d = 0; d < D; ++d) a = fmaf(xr[d], Elem<T>::load(w1e + (int64_t)d * Ed + j), a);
        if (b1 != nullptr) a += Elem<T>::load(b1 + (int64_t)e * Ed + j);
        a = apply_act(act, a);
      } else {
        for (int d = 0; d < D; ++d) {
          a = fmaf(xr[d], Elem<T>::load(w1e + (int64_t)d * Ed + j), a);
          u = fmaf(xr[d], Elem<T>::load(wue + (int64_t)d * Ed + j), u);
        }
        a = apply_act(act, a) * u;
      }
      hs[p] = Elem<T>::round(a) * rs[m * E + e];
    }
    __syncthreads();
    const T* w2e = w2 + (int64_t)e * Ed * D;
    for (int j = 0; j < Ed; ++j) {
      float w[CPT];
#pragma unroll
      for (int c = 0; c < CPT; ++c) {
        const int col = t + c * 256;
        w[c] = (col < D) ? Elem<T>::load(w2e + (int64_t)j * D + col) : 0.f;
      }
#pragma unroll
      for (int m = 0; m < BM; ++m) {
        const float h = hs[m * Ed + j];
#pragma unroll
        for (int c = 0; c < CPT; ++c) acc[m][c] = fmaf(h, w[c], acc[m][c]);
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int col = t + c * 256;
    if (col >= D) continue;
    const float lb = (last_bias != nullptr) ? Elem<T>::load(last_bias + col) : 0.f;
#pragma unroll
    for (int m = 0; m < BM; ++m) {
      const int64_t n = tok0 + m;
      if (n >= N) continue;
      float v = acc[m][c] + lb;
      if (add_residual) v += xs[m * D + col];
      Elem<T>::store(out + n * D + col, v);
    }
  }
}

template <typename T, int BM, int CPT>
static hipError_t launch_experts_generic_cfg(const d2dmoe_shape& sh, const void* x, const void* routing, const void* w1,
                                             const void* b1, const void* w2, const void* w_up, const void* last_bias,
                                             void* out, hipStream_t s) {
  const size_t lds = (size_t)BM * (sh.d_model + sh.n_experts + sh.expert_dim) * sizeof(float) + sh.n_experts * sizeof(int);
  if (lds > 160 * 1024) return hipErrorInvalidValue;
  auto kern = experts_generic_kernel<T, BM, CPT>;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3((unsigned)cdiv64(sh.n_tokens, BM)), dim3(256), lds, s, (const T*)x, (const T*)routing,
                     (const T*)w1, (const T*)b1, (const T*)w2, (const T*)w_up, (const T*)last_bias, (T*)out, sh.n_tokens,
                     sh.d_model, sh.n_experts, sh.expert_dim, sh.activation, sh.add_residual);
  return hipGetLastError();
}

bool experts_generic_supported(const d2dmoe_shape& sh) {
  if (sh.d_model > 4096) return false;
  const int bm = sh.d_model <= 768 ? 16 : (sh.d_model <= 2048 ? 8 : 4);
  const size_t lds = (size_t)bm * (sh.d_model + sh.n_experts + sh.expert_dim) * sizeof(float) + sh.n_experts * sizeof(int);
  return lds <= 160 * 1024;
}

template <typename T>
hipError_t launch_experts_generic(const d2dmoe_shape& sh, const void* x, const void* routing, const void* w1,
                                  const void* b1, const void* w2, const void* w_up, const void* last_bias, void* out,
                                  hipStream_t s) {
  if (sh.d_model <= 768) return launch_experts_generic_cfg<T, 16, 3>(sh, x, routing, w1, b1, w2, w_up, last_bias, out, s);
  if (sh.d_model <= 2048) return launch_experts_generic_cfg<T, 8, 8>(sh, x, routing, w1, b1, w2, w_up, last_bias, out, s);
  return launch_experts_generic_cfg<T, 4, 16>(sh, x, routing, w1, b1, w2, w_up, last_bias, out, s);
}
template hipError_t launch_experts_generic<float>(const d2dmoe_shape&, const void*, const void*, const void*, const void*,
                                                  const void*, const void*, const void*, void*, hipStream_t);
template hipError_t launch_experts_generic<bf16_t>(const d2dmoe_shape&, const void*, const void*, const void*, const void*,
                                                   const void*, const void*, const void*, void*, hipStream_t);
template hipError_t launch_experts_generic<f16_t>(const d2dmoe_shape&, const void*, const void*, const void*, const void*,
                                                   const void*, const void*, const void*, void*, hipStream_t);

}  // namespace d2dmoe
