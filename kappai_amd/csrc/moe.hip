// Mixture of experts: router, the step's rows sorted by expert, the experts' products over that
// order, and the weighted sum.  Nothing is read back by the host: every launch is sized by the
// number of rows alone, so a step with experts can be captured in a graph.
//   moe_route     z = W_router h in float32, the `top` largest chosen (lowest index on ties),
//                 weights = softmax over the chosen logits
//   moe_plan      (row, choice) pairs in expert order, every expert's run starting on a tile of
//                 MOE_TILE_M slots: slot_of_pair, pair_of_slot (-1: empty), tile_expert (-1: unused)
//   moe_gemm      tile by tile: act = silu(x Wg^T) * (x Wu^T) on gathered rows, or y = act Wd^T
//   moe_combine   out[t] = sum_k weight[t, k] * y[slot of (t, k)], in the order of k, float32
#include "common.h"

#define MOE_TILE_M 64          // slots of a tile (the matrix-core kernel: four row tiles of 16)
#define MOE_HALF_M 32          // rows a block of the plain kernel takes: half a tile
#define MOE_TILE_N 64
#define MOE_TILE_K 32
#define MOE_MAX_TOP 16
#define MOE_THREADS 256

extern "C" int kappai_moe_tile_rows() { return MOE_TILE_M; }

#define MOE_ROUTE_GROUP 16      // experts whose sums a thread carries side by side

// A block a row.  The threads stride over the row four columns at a time (one column at a time
// when the width or an address does not allow 16-byte loads), each with the sums of a group of
// experts, whose loads are all asked for before the first is used; the waves' sums meet in LDS
// and are added in the order of the waves.  Then the first wave chooses.
template <typename T, int VEC>
__global__ __launch_bounds__(MOE_THREADS) void moe_route_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ router,
    const float* __restrict__ bias, int n_rows, int D, int E, int top, int* __restrict__ idx,
    float* __restrict__ wts) {
  extern __shared__ float route_lds[];
  constexpr int NW = MOE_THREADS / WAVE;
  float* logits = route_lds;                       // [E]
  float* part = route_lds + E;                     // [MOE_ROUTE_GROUP][NW]
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int row = blockIdx.x;
  const T* xr = x + (size_t)row * ldx;
  for (int e0 = 0; e0 < E; e0 += MOE_ROUTE_GROUP) {
    float acc[MOE_ROUTE_GROUP];
#pragma unroll
    for (int j = 0; j < MOE_ROUTE_GROUP; ++j) acc[j] = 0.f;
    for (int c = threadIdx.x * VEC; c < D; c += MOE_THREADS * VEC) {
      float xv[VEC], rv[MOE_ROUTE_GROUP][VEC];
#pragma unroll
      for (int j = 0; j < MOE_ROUTE_GROUP; ++j) {
        const float* r = router + (size_t)min(e0 + j, E - 1) * D + c;
        if (VEC == 4) {
          const float4 v = *reinterpret_cast<const float4*>(r);
          rv[j][0] = v.x; rv[j][VEC > 1 ? 1 : 0] = v.y; rv[j][VEC > 2 ? 2 : 0] = v.z;
          rv[j][VEC > 3 ? 3 : 0] = v.w;
        } else {
          rv[j][0] = r[0];
        }
      }
#pragma unroll
      for (int i = 0; i < VEC; ++i) xv[i] = to_f32(xr[c + i]);
#pragma unroll
      for (int j = 0; j < MOE_ROUTE_GROUP; ++j)
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[j] = fmaf(xv[i], rv[j][i], acc[j]);
    }
#pragma unroll
    for (int j = 0; j < MOE_ROUTE_GROUP; ++j) {
      const float sum = wave_sum(acc[j]);
      if (lane == 0) part[j * NW + wave] = sum;
    }
    __syncthreads();
    if (threadIdx.x < MOE_ROUTE_GROUP && e0 + threadIdx.x < E) {
      float sum = part[threadIdx.x * NW];
      for (int w = 1; w < NW; ++w) sum += part[threadIdx.x * NW + w];
      logits[e0 + threadIdx.x] = bias ? sum + bias[e0 + threadIdx.x] : sum;
    }
    __syncthreads();
  }
  if (wave != 0) return;
  float cv[MOE_MAX_TOP];
  int ci[MOE_MAX_TOP];
#pragma unroll
  for (int k = 0; k < MOE_MAX_TOP; ++k) {
    if (k < top) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int e = lane; e < E; e += WAVE) {
        const float v = logits[e];
        if (v > best) { best = v; at = e; }      // the lowest index among a lane's equals
      }
      const float m = wave_max(best);
      const int who = -wave_max(best == m ? -at : -0x7fffffff);
      cv[k] = m;
      ci[k] = who;
      __builtin_amdgcn_wave_barrier();
      if (lane == 0 && who < E) logits[who] = -INFINITY;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (lane == 0) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < MOE_MAX_TOP; ++k)
      if (k < top) sum += expf(cv[k] - cv[0]);
#pragma unroll
    for (int k = 0; k < MOE_MAX_TOP; ++k)
      if (k < top) {
        idx[(size_t)row * top + k] = ci[k] < E ? ci[k] : 0;
        wts[(size_t)row * top + k] = expf(cv[k] - cv[0]) / sum;
      }
  }
}

extern "C" int kappai_moe_route(const void* x, int ldx, int x_is_bf16, const float* router,
                                const float* bias, int T, int D, int E, int top, int* idx,
                                float* wts, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || top > MOE_MAX_TOP || top > E || E > 4096) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(E + MOE_ROUTE_GROUP * (MOE_THREADS / WAVE)) * sizeof(float);
  const bool vec = D % 4 == 0 && (uintptr_t)router % 16 == 0;
#define MOE_ROUTE_LAUNCH(TT, V)                                                                 \
  hipLaunchKernelGGL((moe_route_kernel<TT, V>), dim3(T), dim3(MOE_THREADS), lds, stream,          \
                     (const TT*)x, ldx, router, bias, T, D, E, top, idx, wts)
  if (x_is_bf16) {
    if (vec) MOE_ROUTE_LAUNCH(bf16_t, 4); else MOE_ROUTE_LAUNCH(bf16_t, 1);
  } else {
    if (vec) MOE_ROUTE_LAUNCH(float, 4); else MOE_ROUTE_LAUNCH(float, 1);
  }
#undef MOE_ROUTE_LAUNCH
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// The pairs sorted by expert, stably and without atomics.  The waves of one block each take a
// run of the pairs, 64 at a time: the lanes with the same expert are found by ballots and placed
// by counting the lanes below.  Pass 1 counts per wave and expert; then every expert's run gets
// its first slot (a multiple of MOE_TILE_M) and every wave its place in the run; pass 2 places.
#define MOE_PLAN_MAX_WAVES 16

__device__ __forceinline__ void moe_plan_pass(const int* __restrict__ idx, int p_lo, int p_hi,
                                              int* cnt, const int* start, bool place,
                                              int* __restrict__ slot_of_pair,
                                              int* __restrict__ pair_of_slot) {
  const int lane = threadIdx.x % WAVE;
  for (int p0 = p_lo; p0 < p_hi; p0 += WAVE) {
    const int p = p0 + lane;
    const int e = p < p_hi ? idx[p] : -1;
    bool todo = p < p_hi;
    while (true) {
      const unsigned long long rest = __ballot(todo);
      if (!rest) break;
      const int cur = __shfl(e, __ffsll((long long)rest) - 1);
      const bool mine = todo && e == cur;
      const unsigned long long mask = __ballot(mine);
      const int before = cnt[cur];          // (only this wave writes its counters)
      if (place && mine) {
        const int slot = start[cur] + before + __popcll(mask & ((1ull << lane) - 1ull));
        slot_of_pair[p] = slot;
        pair_of_slot[slot] = p;
      }
      __builtin_amdgcn_wave_barrier();
      if (lane == 0) cnt[cur] = before + __popcll(mask);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (mine) todo = false;
    }
  }
}

__global__ __launch_bounds__(MOE_PLAN_MAX_WAVES * WAVE) void moe_plan_kernel(
    const int* __restrict__ idx, int P, int E, int n_tiles, int n_waves,
    int* __restrict__ slot_of_pair, int* __restrict__ pair_of_slot,
    int* __restrict__ tile_expert) {
  extern __shared__ int plan_lds[];
  int* base = plan_lds;                 // [E] first slot of the expert's run
  int* len = plan_lds + E;              // [E] pairs of the expert
  int* cnt = plan_lds + 2 * E;          // [n_waves][E] pairs of the wave; then placed so far
  int* start = cnt + n_waves * E;       // [n_waves][E] first slot of the wave's pairs of e
  const int tid = threadIdx.x, nt = blockDim.x;
  const int wave = tid / WAVE;
  for (int i = tid; i < n_waves * E; i += nt) cnt[i] = 0;
  for (int i = tid; i < n_tiles * MOE_TILE_M; i += nt) pair_of_slot[i] = -1;
  for (int i = tid; i < n_tiles; i += nt) tile_expert[i] = -1;
  __syncthreads();
  const int per = ((P + n_waves * WAVE - 1) / (n_waves * WAVE)) * WAVE;
  const int p_lo = min(P, wave * per), p_hi = min(P, p_lo + per);
  moe_plan_pass(idx, p_lo, p_hi, cnt + wave * E, nullptr, false, slot_of_pair, pair_of_slot);
  __syncthreads();
  // the runs' lengths and, inside a run, the waves one after the other
  for (int e = tid; e < E; e += nt) {
    int sum = 0;
    for (int w = 0; w < n_waves; ++w) {
      const int c = cnt[w * E + e];
      start[w * E + e] = sum;
      sum += c;
      cnt[w * E + e] = 0;
    }
    len[e] = sum;
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      base[e] = at;
      at += (len[e] + MOE_TILE_M - 1) / MOE_TILE_M * MOE_TILE_M;
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += nt) {
    const int first = base[e];
    for (int w = 0; w < n_waves; ++w) start[w * E + e] += first;
    const int n = (len[e] + MOE_TILE_M - 1) / MOE_TILE_M;
    for (int i = 0; i < n; ++i) tile_expert[first / MOE_TILE_M + i] = e;
  }
  __syncthreads();
  moe_plan_pass(idx, p_lo, p_hi, cnt + wave * E, start + wave * E, true, slot_of_pair,
                pair_of_slot);
}

extern "C" int kappai_moe_plan(const int* idx, int P, int E, int n_tiles, int* slot_of_pair,
                               int* pair_of_slot, int* tile_expert, hipStream_t stream) {
  if (P <= 0) return 0;
  if (E < 1 || E > 4096 || n_tiles < P / MOE_TILE_M + (E < P ? E : P))
    return (int)hipErrorInvalidValue;
  // as many waves as have 64 pairs each and as the counters of fit into 48 KB of LDS
  int n_waves = (P + WAVE - 1) / WAVE;
  if (n_waves > MOE_PLAN_MAX_WAVES) n_waves = MOE_PLAN_MAX_WAVES;
  while (n_waves > 1 && (size_t)(2 * n_waves + 2) * E * sizeof(int) > 48 * 1024) --n_waves;
  const size_t lds = (size_t)(2 * n_waves + 2) * E * sizeof(int);
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(n_waves * WAVE), lds, stream, idx, P, E,
                     n_tiles, n_waves, slot_of_pair, pair_of_slot, tile_expert);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

__device__ __forceinline__ float silu_exact(float g) { return g / (1.0f + expf(-g)); }
__device__ __forceinline__ float relu_squared(float z) { const float r = fmaxf(z, 0.f); return r * r; }

// Half a tile (MOE_HALF_M slots) of one expert times MOE_TILE_N rows of its matrix, float sums on
// the vector units (this is the 32-bit path, and the path of any shape).  GATED: the rows are
// gathered from x by pair / top, two matrices, out = silu(g) * u in T; GATED == 2: gathered rows,
// one matrix, out = relu(x W^T)^2 in T; else the rows are the slots of `a` themselves and out is
// float.
template <typename T, int GATED>
__global__ __launch_bounds__(MOE_THREADS) void moe_gemm_kernel(
    const T* __restrict__ a, int lda, const T* __restrict__ w0, const T* __restrict__ w1, int N,
    int K, const int* __restrict__ tile_expert, const int* __restrict__ pair_of_slot, int top,
    void* __restrict__ out_v) {
  const int tile = blockIdx.x / 2, slot0 = blockIdx.x * MOE_HALF_M;
  const int e = tile_expert[tile];
  if (e < 0) return;
  __shared__ float As[MOE_TILE_K][MOE_HALF_M + 1];
  __shared__ float W0s[MOE_TILE_K][MOE_TILE_N + 1];
  __shared__ float W1s[GATED == 1 ? MOE_TILE_K : 1][MOE_TILE_N + 1];
  __shared__ int src_row[MOE_HALF_M];
  const int tid = threadIdx.x;
  if (tid < MOE_HALF_M) {
    const int slot = slot0 + tid;
    const int pair = pair_of_slot[slot];
    src_row[tid] = pair < 0 ? -1 : (GATED ? pair / top : slot);
  }
  __syncthreads();
  const int n0 = blockIdx.y * MOE_TILE_N;
  const T* W0 = w0 + (size_t)e * N * K;
  const T* W1 = GATED == 1 ? w1 + (size_t)e * N * K : nullptr;
  const int ty = tid / 16, tx = tid % 16;
  float acc0[2][4] = {}, acc1[2][4] = {};
  const int am = tid / 8, ak = (tid % 8) * 4;       // this thread's piece of the A tile
  const int wn = tid / 4, wk = (tid % 4) * 8;       // and of the W tiles
  for (int k0 = 0; k0 < K; k0 += MOE_TILE_K) {
    const int r = src_row[am];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + ak + i;
      As[ak + i][am] = (r >= 0 && k < K) ? to_f32(a[(size_t)r * lda + k]) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + wk + i, n = n0 + wn;
      const bool ok = n < N && k < K;
      W0s[wk + i][wn] = ok ? to_f32(W0[(size_t)n * K + k]) : 0.f;
      if (GATED == 1) W1s[wk + i][wn] = ok ? to_f32(W1[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < MOE_TILE_K; ++k) {
      const float a0 = As[k][2 * ty], a1 = As[k][2 * ty + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b0 = W0s[k][tx + 16 * j];
        acc0[0][j] = fmaf(a0, b0, acc0[0][j]);
        acc0[1][j] = fmaf(a1, b0, acc0[1][j]);
        if (GATED == 1) {
          const float b1 = W1s[k][tx + 16 * j];
          acc1[0][j] = fmaf(a0, b1, acc1[0][j]);
          acc1[1][j] = fmaf(a1, b1, acc1[1][j]);
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = 2 * ty + i;
    if (src_row[m] < 0) continue;
    const size_t slot = (size_t)slot0 + m;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      if (GATED == 1)
        from_f32((T*)out_v + slot * N + n, silu_exact(acc0[i][j]) * acc1[i][j]);
      else if (GATED == 2)
        from_f32((T*)out_v + slot * N + n, relu_squared(acc0[i][j]));
      else
        ((float*)out_v)[slot * N + n] = acc0[i][j];
    }
  }
}

extern "C" int kappai_moe_gemm(const void* a, int lda, const void* w0, const void* w1, int N,
                               int K, const int* tile_expert, const int* pair_of_slot, int top,
                               int n_tiles, void* out, int gated, int is_bf16,
                               hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  const dim3 grid(n_tiles * (MOE_TILE_M / MOE_HALF_M), (N + MOE_TILE_N - 1) / MOE_TILE_N);
  if (grid.y > 65535) return (int)hipErrorInvalidValue;
#define MOE_GEMM_LAUNCH(TT, G)                                                                  \
  hipLaunchKernelGGL((moe_gemm_kernel<TT, G>), grid, dim3(MOE_THREADS), 0, stream, (const TT*)a, \
                     lda, (const TT*)w0, (const TT*)w1, N, K, tile_expert, pair_of_slot, top, out)
  if (gated < 0 || gated > 2) return (int)hipErrorInvalidValue;
  if (is_bf16) {
    if (gated == 1) MOE_GEMM_LAUNCH(bf16_t, 1); else if (gated == 2) MOE_GEMM_LAUNCH(bf16_t, 2);
    else MOE_GEMM_LAUNCH(bf16_t, 0);
  } else {
    if (gated == 1) MOE_GEMM_LAUNCH(float, 1); else if (gated == 2) MOE_GEMM_LAUNCH(float, 2);
    else MOE_GEMM_LAUNCH(float, 0);
  }
#undef MOE_GEMM_LAUNCH
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// The same products in bfloat16 on the matrix cores (v_mfma_f32_16x16x32_bf16).  A block owns a
// tile of 64 slots (four row tiles of 16) and 4 waves x NT column tiles of 16 rows of the
// expert's matrices; a wave streams its rows of W (and of the second matrix when GATED) and the
// tile's activation rows straight from memory into registers, 16 bytes a lane, the next step of
// 32 of K on its way while this one is multiplied.  Lane l holds row l % 16 of a fragment and the eight values of K from
// 8 (l / 16); of a result tile it holds column l % 16 and the rows 4 (l / 16) .. + 3.
// K must be a multiple of 8 and every row 16-byte aligned (fragment order: K a multiple of 32,
// the matrices' rows a multiple of 16).
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t moe_u32x4_t;

#define MOE_MFMA_WAVES 4

// WF: the experts' matrices lie in fragment order (the host arranges them once): the 16 rows x
// 32 of K that a matrix instruction takes are 1 KB in a row, lane after lane, tile (row tile,
// step of K) after tile, so that a wave's load is one piece of memory instead of sixteen.
// BYROW: the block's four waves take four tiles in a row and the same columns (a step of many
// rows: tiles in a row mostly belong to one expert, whose matrix the waves then read together,
// once a block instead of once a tile); else they take one tile and four sets of columns.
template <int GATED, int NT, int U, bool WF, bool BYROW>
__global__ __launch_bounds__(MOE_MFMA_WAVES * WAVE) void moe_gemm_mfma_kernel(
    const bf16_t* __restrict__ a, int lda, const bf16_t* __restrict__ w0,
    const bf16_t* __restrict__ w1, int N, int K, const int* __restrict__ tile_expert,
    const int* __restrict__ pair_of_slot, int top, int n_tiles, void* __restrict__ out_v) {
  constexpr int MT = MOE_TILE_M / 16;
  constexpr int NG = GATED == 1 ? 2 : 1;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int tile = BYROW ? blockIdx.x * MOE_MFMA_WAVES + wave : blockIdx.x;
  if (tile >= n_tiles) return;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int col = lane % 16, kg = 8 * (lane / 16);
  const int n0 = BYROW ? blockIdx.y * 16 * NT : (blockIdx.y * MOE_MFMA_WAVES + wave) * 16 * NT;
  if (n0 >= N) return;
  const bf16_t* arow[MT];
  bool a_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int slot = tile * MOE_TILE_M + t * 16 + col;
    const int pair = pair_of_slot[slot];
    a_ok[t] = pair >= 0;
    const int r = pair < 0 ? 0 : (GATED ? pair / top : slot);
    arow[t] = a + (size_t)r * lda + kg;
  }
  const bf16_t* wrow[NG][NT];
  bool w_ok[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n0 + 16 * j + col;
    w_ok[j] = n < N;
    const size_t at = WF ? (size_t)e * N * K + (size_t)((w_ok[j] ? n : 0) / 16) * (K / 32) * 512 +
                               lane * 8
                         : ((size_t)e * N + (w_ok[j] ? n : 0)) * K + kg;
    wrow[0][j] = w0 + at;
    if (GATED == 1) wrow[1][j] = w1 + at;
  }
  moe_f32x4_t acc[NG][NT][MT];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[g][j][t] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
  const moe_u32x4_t zero = {0u, 0u, 0u, 0u};
  // the loads of the next U steps of 32 of K are on their way while these are multiplied
  moe_u32x4_t av[2][U][MT], wv[2][U][NG][NT];
  auto load = [&](int buf, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int gk = k0 + 32 * u;
      const bool kin = gk + kg < K;
#pragma unroll
      for (int t = 0; t < MT; ++t)
        av[buf][u][t] =
            (kin && a_ok[t]) ? *reinterpret_cast<const moe_u32x4_t*>(arow[t] + gk) : zero;
#pragma unroll
      for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          wv[buf][u][g][j] = (kin && w_ok[j])
                                 ? *reinterpret_cast<const moe_u32x4_t*>(
                                       wrow[g][j] + (WF ? (size_t)(gk / 32) * 512 : (size_t)gk))
                                 : zero;
    }
  };
  auto multiply = [&](int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int t = 0; t < MT; ++t)
            acc[g][j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(moe_bf16x8_t, av[buf][u][t]),
                __builtin_bit_cast(moe_bf16x8_t, wv[buf][u][g][j]), acc[g][j][t], 0, 0, 0);
  };
  load(0, 0);
  for (int k = 0; k < K; k += 64 * U) {
    load(1, k + 32 * U);
    multiply(0);
    load(0, k + 64 * U);
    multiply(1);
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int m = t * 16 + 4 * (lane / 16) + v;
      const size_t slot = (size_t)tile * MOE_TILE_M + m;
      if (pair_of_slot[slot] < 0) continue;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int n = n0 + 16 * j + col;
        if (n >= N) continue;
        if (GATED == 1)
          ((bf16_t*)out_v)[slot * N + n] =
              f32_to_bf16(silu_exact(acc[0][j][t][v]) * acc[GATED == 1 ? 1 : 0][j][t][v]);
        else if (GATED == 2)
          ((bf16_t*)out_v)[slot * N + n] = f32_to_bf16(relu_squared(acc[0][j][t][v]));
        else
          ((float*)out_v)[slot * N + n] = acc[0][j][t][v];
      }
    }
}

// `few`: a step of few rows (decoding), where a tile holds a row or two and the kernel streams
// the experts' matrices: one column tile a wave (twice the blocks) and two steps of K a load.
extern "C" int kappai_moe_gemm_mfma(const void* a, int lda, const void* w0, const void* w1, int N,
                                    int K, const int* tile_expert, const int* pair_of_slot,
                                    int top, int n_tiles, void* out, int gated, int few,
                                    int w_frag, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if ((K % 8) || (lda % 8) || ((uintptr_t)a % 16) || ((uintptr_t)w0 % 16) || ((uintptr_t)w1 % 16))
    return (int)hipErrorInvalidValue;
  if (w_frag && ((K % 32) || (N % 16))) return (int)hipErrorInvalidValue;
  const dim3 block(MOE_MFMA_WAVES * WAVE);
#define MOE_MFMA_LAUNCH(G, NT_, U_, BR_)                                                         \
  if (w_frag) MOE_MFMA_LAUNCH_WF(G, NT_, U_, true, BR_); else MOE_MFMA_LAUNCH_WF(G, NT_, U_, false, BR_)
#define MOE_MFMA_LAUNCH_WF(G, NT_, U_, WF_, BR_)                                                 \
  hipLaunchKernelGGL(                                                                            \
      (moe_gemm_mfma_kernel<G, NT_, U_, WF_, BR_>),                                              \
      BR_ ? dim3((n_tiles + MOE_MFMA_WAVES - 1) / MOE_MFMA_WAVES, (N + 16 * NT_ - 1) / (16 * NT_)) \
          : dim3(n_tiles, (N + 16 * NT_ * MOE_MFMA_WAVES - 1) / (16 * NT_ * MOE_MFMA_WAVES)),      \
      block, 0, stream, (const bf16_t*)a, lda, (const bf16_t*)w0, (const bf16_t*)w1, N, K,         \
      tile_expert, pair_of_slot, top, n_tiles, out)
  if (gated < 0 || gated > 2) return (int)hipErrorInvalidValue;
  if (gated == 1) {
    if (few) { MOE_MFMA_LAUNCH(1, 1, 2, false); } else { MOE_MFMA_LAUNCH(1, 4, 1, true); }
  } else if (gated == 2) {
    if (few) { MOE_MFMA_LAUNCH(2, 2, 2, false); } else { MOE_MFMA_LAUNCH(2, 4, 1, true); }
  } else {
    if (few) { MOE_MFMA_LAUNCH(0, 2, 2, false); } else { MOE_MFMA_LAUNCH(0, 4, 1, true); }
  }
#undef MOE_MFMA_LAUNCH
#undef MOE_MFMA_LAUNCH_WF
  KAPPAI_RETURN_LAUNCH_STATUS();
}

__global__ __launch_bounds__(MOE_THREADS) void moe_combine_kernel(
    const float* __restrict__ y, const int* __restrict__ slot_of_pair,
    const float* __restrict__ wts, int top, int D, const void* __restrict__ also,
    int also_is_bf16, int also_parts, size_t also_plane, float* __restrict__ out) {
  const int t = blockIdx.x;
  for (int n = blockIdx.y * MOE_THREADS + threadIdx.x; n < D; n += gridDim.y * MOE_THREADS) {
    // what every row gets beside its experts (a shared expert's result: rows, or float planes
    // of a product cut over its input dimension, added in order) comes first
    float acc = 0.f;
    if (also != nullptr) {
      const size_t at = (size_t)t * D + n;
      if (also_is_bf16) acc = bf16_to_f32(((const bf16_t*)also)[at]);
      else
        for (int p = 0; p < also_parts; ++p) acc += ((const float*)also)[p * also_plane + at];
    }
    for (int k = 0; k < top; ++k)
      acc = fmaf(wts[(size_t)t * top + k], y[(size_t)slot_of_pair[(size_t)t * top + k] * D + n],
                 acc);
    out[(size_t)t * D + n] = acc;
  }
}

extern "C" int kappai_moe_combine(const float* y, const int* slot_of_pair, const float* wts, int T,
                                  int top, int D, const void* also, int also_is_bf16,
                                  int also_parts, float* out, hipStream_t stream) {
  if (T <= 0) return 0;
  if (also && also_parts < 1) return (int)hipErrorInvalidValue;
  // few rows: a thread a column, so that all its loads are asked for at once
  const int col_blocks = T <= 512 ? min(64, (D + MOE_THREADS - 1) / MOE_THREADS) : 1;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T, col_blocks), dim3(MOE_THREADS), 0, stream, y, slot_of_pair,
                     wts, top, D, also, also_is_bf16, also_parts, (size_t)T * D, out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
