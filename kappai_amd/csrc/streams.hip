// A residual stream kept in several copies ("hyper-connections"), the layer norm that reads it,
// and small gates and caps around attention layers that use them.
//
//   hyper_step     one pass over a row's S copies x_1 .. x_S [T, S, W] (float32):
//                    write:  x_t <- sum_s mix[s, t] x_s + out[t] * y     (all t from the old x_s)
//                    read:   u = sum_s in[s] x_s;  rows = (u - mean) / sqrt(var + eps) * w
//                  either half may be left out; `source`: the copies do not exist yet and are all
//                  that row [T, W] (the embedded rows); `rows`: only the listed rows
//                  are read (and, with a write half, their new copies are not stored: the norm
//                  before the output head).
//   rows_rmsnorm   y = x / sqrt(mean(x^2) + eps) * w on the first n columns of strided rows
//   sigmoid_gate   x[t, i] *= sigmoid(g[t, i / group])
//   softcap_rows   x <- c tanh(x / c), in place, float32
//   activate       out = relu(x)^2 (kind 0)
#include "common.h"

#define HS_THREADS 256          // threads of a block when there are rows enough to fill the chip
#define HS_MAX_THREADS 1024     // with few rows a block is as wide as the row has pieces
#define HS_MAX_STREAMS 8

// VEC values of an update from column c on: rows of TY, or P float planes [P, T, W] added in order
template <int VEC>
__device__ __forceinline__ void update_at(const float* __restrict__ y, int parts, size_t plane,
                                          size_t at, float* v) {
  // four planes are asked for at once and added in their order (a loop that waits for every
  // plane before it asks for the next costs a trip to memory a plane)
  if (VEC == 4) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int p0 = 0; p0 < parts; p0 += 4) {
      float4 b[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        b[j] = p0 + j < parts ? *reinterpret_cast<const float4*>(y + (size_t)(p0 + j) * plane + at)
                              : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (p0 + j == 0) acc = b[j];
        else if (p0 + j < parts) { acc.x += b[j].x; acc.y += b[j].y; acc.z += b[j].z; acc.w += b[j].w; }
      }
    }
    v[0] = acc.x; v[VEC > 1 ? 1 : 0] = acc.y; v[VEC > 2 ? 2 : 0] = acc.z; v[VEC > 3 ? 3 : 0] = acc.w;
  } else {
    v[0] = y[at];
    for (int p = 1; p < parts; ++p) v[0] += y[(size_t)p * plane + at];
  }
}
template <int VEC>
__device__ __forceinline__ void update_at(const bf16_t* __restrict__ y, int, size_t, size_t at,
                                          float* v) {
  if (VEC == 4) {
    const uint2 a = *reinterpret_cast<const uint2*>(y + at);
    v[0] = __uint_as_float(a.x << 16);
    v[VEC > 1 ? 1 : 0] = __uint_as_float(a.x & 0xffff0000u);
    v[VEC > 2 ? 2 : 0] = __uint_as_float(a.y << 16);
    v[VEC > 3 ? 3 : 0] = __uint_as_float(a.y & 0xffff0000u);
  } else {
    v[0] = bf16_to_f32(y[at]);
  }
}

template <int VEC>
__device__ __forceinline__ void load_f32(const float* p, float* v) {
  if (VEC == 4) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    v[0] = a.x; v[VEC > 1 ? 1 : 0] = a.y; v[VEC > 2 ? 2 : 0] = a.z; v[VEC > 3 ? 3 : 0] = a.w;
  } else {
    v[0] = p[0];
  }
}
template <int VEC>
__device__ __forceinline__ void store_f32(float* p, const float* v) {
  if (VEC == 4)
    *reinterpret_cast<float4*>(p) =
        make_float4(v[0], v[VEC > 1 ? 1 : 0], v[VEC > 2 ? 2 : 0], v[VEC > 3 ? 3 : 0]);
  else
    p[0] = v[0];
}
template <int VEC>
__device__ __forceinline__ void store_rows(float* p, const float* v) { store_f32<VEC>(p, v); }
template <int VEC>
__device__ __forceinline__ void store_rows(bf16_t* p, const float* v) {
  if (VEC == 4)
    *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v[0], v[VEC > 1 ? 1 : 0]),
                                              pack_bf16x2(v[VEC > 2 ? 2 : 0], v[VEC > 3 ? 3 : 0]));
  else
    p[0] = f32_to_bf16(v[0]);
}

// A block a row; a thread takes VEC neighbouring columns at a time (VEC 4: 16-byte loads and
// stores; the width and every address then are multiples of four values).  The weights among the
// copies go through LDS once a block.
template <typename TY, typename TO, int VEC, int MAXT>
__global__ __launch_bounds__(MAXT) void hyper_step_kernel(
    float* __restrict__ streams, const float* __restrict__ source, const TY* __restrict__ y,
    int parts, const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, const float* __restrict__ norm_w, float eps,
    const int* __restrict__ rows, int store, TO* __restrict__ normed, int T, int S, int W) {
  extern __shared__ float hs_lds[];
  float* u_row = hs_lds;                 // [W]
  float* red = hs_lds + W;               // [16]
  const int t = rows ? rows[blockIdx.x] : blockIdx.x;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const bool write = y != nullptr, read = normed != nullptr;
  __shared__ float c_mix[HS_MAX_STREAMS * HS_MAX_STREAMS], c_out[HS_MAX_STREAMS],
      c_in[HS_MAX_STREAMS];
  if (tid < S * S && write) c_mix[tid] = mix[tid];
  if (tid < S && write) c_out[tid] = out_w[tid];
  if (tid < S && read) c_in[tid] = in_w[tid];
  __syncthreads();
  // the norm's weights for this thread's first columns are asked for with the row itself
  float w_first[VEC];
  const bool has_first = read && tid * VEC < W;
  if (has_first) load_f32<VEC>(norm_w + tid * VEC, w_first);
  const size_t plane = (size_t)T * W;
  float sum = 0.f;
  for (int c = tid * VEC; c < W; c += nthreads * VEC) {
    float x[HS_MAX_STREAMS][VEC];
#pragma unroll
    for (int s = 0; s < HS_MAX_STREAMS; ++s)
      if (s < S)
        load_f32<VEC>(source ? source + (size_t)t * W + c : streams + ((size_t)t * S + s) * W + c,
                      x[s]);
    if (write) {
      float yv[VEC];
      update_at<VEC>(y, parts, plane, (size_t)t * W + c, yv);
      float nx[HS_MAX_STREAMS][VEC];
#pragma unroll
      for (int to = 0; to < HS_MAX_STREAMS; ++to)
        if (to < S) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < HS_MAX_STREAMS; ++s)
              if (s < S) acc = fmaf(c_mix[s * S + to], x[s][i], acc);
            nx[to][i] = fmaf(c_out[to], yv[i], acc);
          }
        }
#pragma unroll
      for (int s = 0; s < HS_MAX_STREAMS; ++s)
        if (s < S) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) x[s][i] = nx[s][i];
          if (store) store_f32<VEC>(streams + ((size_t)t * S + s) * W + c, nx[s]);
        }
    } else if (source && store) {
#pragma unroll
      for (int s = 0; s < HS_MAX_STREAMS; ++s)
        if (s < S) store_f32<VEC>(streams + ((size_t)t * S + s) * W + c, x[s]);
    }
    if (read) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < HS_MAX_STREAMS; ++s)
          if (s < S) u = fmaf(c_in[s], x[s][i], u);
        u_row[c + i] = u;
        sum += u;
      }
    }
  }
  if (!read) return;
  const float mean = block_sum(sum, red) / (float)W;
  float sq = 0.f;
  for (int c = tid * VEC; c < W; c += nthreads * VEC) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float d = u_row[c + i] - mean;
      sq = fmaf(d, d, sq);
    }
  }
  const float rstd = 1.0f / sqrtf(block_sum(sq, red) / (float)W + eps);
  TO* dst = normed + (size_t)blockIdx.x * W;
  for (int c = tid * VEC; c < W; c += nthreads * VEC) {
    float o[VEC], w[VEC];
    if (c == tid * VEC) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) w[i] = w_first[i];
    } else {
      load_f32<VEC>(norm_w + c, w);
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = (u_row[c + i] - mean) * rstd * w[i];
    store_rows<VEC>(dst + c, o);
  }
}

extern "C" int kappai_hyper_step(float* streams, const float* source, const void* y,
                                 int y_is_bf16, int parts, const float* mix, const float* out_w,
                                 const float* in_w, const float* norm_w, float eps,
                                 const int* rows, int n_rows, int store, void* normed,
                                 int normed_is_bf16, int T, int S, int W, hipStream_t stream) {
  const int blocks = rows ? n_rows : T;
  if (blocks <= 0) return 0;
  if (S < 1 || S > HS_MAX_STREAMS || W < 1 || parts < 1 || (!streams && !source) ||
      (y && (!mix || !out_w)) || (normed && (!in_w || !norm_w)) || (store && !streams) ||
      (rows && store))
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(W + 16) * sizeof(float);
  if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
  const bool vec = W % 4 == 0 && ((uintptr_t)streams | (uintptr_t)source | (uintptr_t)norm_w |
                                  (uintptr_t)normed) % 16 == 0 && (uintptr_t)y % 16 == 0;
  // few rows: every piece of the row has a thread of its own, so all its loads are asked for at
  // once (a step of single tokens waits for memory, not for bandwidth)
  int threads = HS_THREADS;
  if (blocks <= 512) {
    const int pieces = (W + (vec ? 4 : 1) - 1) / (vec ? 4 : 1);
    threads = min(HS_MAX_THREADS, max(WAVE, (pieces + WAVE - 1) / WAVE * WAVE));
  }
#define HS_LAUNCH_V(TY, TO, V, MT)                                                               \
  hipLaunchKernelGGL((hyper_step_kernel<TY, TO, V, MT>), dim3(blocks), dim3(threads), lds, stream, \
                     streams, source, (const TY*)y, parts, mix, out_w, in_w, norm_w, eps, rows,   \
                     store, (TO*)normed, T, S, W)
#define HS_LAUNCH(TY, TO)                                                                        \
  if (threads > HS_THREADS) {                                                                    \
    if (vec) HS_LAUNCH_V(TY, TO, 4, HS_MAX_THREADS); else HS_LAUNCH_V(TY, TO, 1, HS_MAX_THREADS); \
  } else {                                                                                       \
    if (vec) HS_LAUNCH_V(TY, TO, 4, HS_THREADS); else HS_LAUNCH_V(TY, TO, 1, HS_THREADS);         \
  }
  if (y_is_bf16) {
    if (normed_is_bf16) { HS_LAUNCH(bf16_t, bf16_t); } else { HS_LAUNCH(bf16_t, float); }
  } else {
    if (normed_is_bf16) { HS_LAUNCH(float, bf16_t); } else { HS_LAUNCH(float, float); }
  }
#undef HS_LAUNCH
#undef HS_LAUNCH_V
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// A block a row: the first n columns of a row of `x` (stride ldx), normed into `out` [T, n].
template <typename T>
__global__ __launch_bounds__(256) void rows_rmsnorm_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ w, float eps, int n,
    T* __restrict__ out) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  const T* xr = x + (size_t)row * ldx;
  float sq = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = to_f32(xr[c]);
    sq = fmaf(v, v, sq);
  }
  const float r = 1.0f / sqrtf(block_sum(sq, red) / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x)
    from_f32(out + (size_t)row * n + c, to_f32(xr[c]) * r * w[c]);
}

extern "C" int kappai_rows_rmsnorm(const void* x, int ldx, const float* w, float eps, int T,
                                   int n, void* out, int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (n < 1 || ldx < n) return (int)hipErrorInvalidValue;
  const dim3 grid(T), block(n <= 64 ? 64 : n <= 128 ? 128 : 256);
  if (is_bf16)
    hipLaunchKernelGGL(rows_rmsnorm_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, ldx,
                       w, eps, n, (bf16_t*)out);
  else
    hipLaunchKernelGGL(rows_rmsnorm_kernel<float>, grid, block, 0, stream, (const float*)x, ldx, w,
                       eps, n, (float*)out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ x, const T* __restrict__ g, int ldg, int n,
                                    int group, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / n;
  const int c = (int)(i - t * n);
  const float z = to_f32(g[t * ldg + c / group]);
  from_f32(x + i, to_f32(x[i]) / (1.0f + expf(-z)));
}

extern "C" int kappai_sigmoid_gate(void* x, const void* g, int ldg, int T, int n, int group,
                                   int is_bf16, hipStream_t stream) {
  const size_t total = (size_t)T * n;
  if (total == 0) return 0;
  if (group < 1 || n % group) return (int)hipErrorInvalidValue;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (is_bf16)
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                       (bf16_t*)x, (const bf16_t*)g, ldg, n, group, total);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, dim3(blocks), dim3(256), 0, stream, (float*)x,
                       (const float*)g, ldg, n, group, total);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

__global__ void softcap_rows_kernel(float* __restrict__ x, float cap, float inv, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] * inv);
}

extern "C" int kappai_softcap_rows(float* x, long n, float cap, hipStream_t stream) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(softcap_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                     x, cap, 1.0f / cap, (size_t)n);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

template <typename T>
__global__ void activate_kernel(const T* __restrict__ in, T* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float r = fmaxf(to_f32(in[i]), 0.f);
  from_f32(out + i, r * r);
}

extern "C" int kappai_activate(const void* in, void* out, long n, int kind, int is_bf16,
                               hipStream_t stream) {
  if (n <= 0) return 0;
  if (kind != 0) return (int)hipErrorInvalidValue;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (is_bf16)
    hipLaunchKernelGGL(activate_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                       (const bf16_t*)in, (bf16_t*)out, (size_t)n);
  else
    hipLaunchKernelGGL(activate_kernel<float>, dim3(blocks), dim3(256), 0, stream,
                       (const float*)in, (float*)out, (size_t)n);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
