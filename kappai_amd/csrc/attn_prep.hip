// What stands between an attention layer's projections and the paged attention kernels when the
// layer is not the plain grouped-query form: queries, keys and values are normalised, scaled,
// rotated and laid out as heads of one size D (zeros behind what a head really holds), keys go to
// the key pool [page][kv_head][slot][D], values transposed to [page][kv_head][D][slot].
//
//   projection_norm_store   RMS norm over the WHOLE q projection (all heads at once) and over the
//                           whole k projection, a query factor that grows with the position,
//                           heads of d (q, k) and dv (v) widened to D
//   latent_store            keys and values from one latent vector a token: the normalised latent
//                           c [r] and a rotated part [rot] shared by all heads become the one kv
//                           head's key [c | rot | 0]; c again is its value; the queries' rotated
//                           parts are rotated and put behind the r places that the product with
//                           the keys' up-projection fills (headwise_linear)
//   headwise_linear         y[t, h, :] = W[h] x[t, h, :], a matrix per head
//   head_norm_rotate_store  RMS norm of every q and k head by itself (one weight [d] for all
//                           heads), rotation of the first places, heads of d and dv widened to D
#include "common.h"

#define AP_THREADS 256

// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(AP_THREADS) void projection_norm_store_kernel(
    const T* __restrict__ proj, int stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, float temp_coef, int temp_every,
    T* __restrict__ k_pool, T* __restrict__ v_pool, const int* __restrict__ row_pos,
    const int* __restrict__ row_seg, const int* __restrict__ block_tables, int max_blocks, int H,
    int G, int d, int dv, int D, int ps, T* __restrict__ q_out) {
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int pos = row_pos[t];
  const T* row = proj + (size_t)t * stride;
  const int nq = H * d, nk = G * d;
  float fq = 1.f, fk = 1.f;
  if (q_norm_w != nullptr) {
    float ss = 0.f;
    for (int e = tid; e < nq; e += AP_THREADS) { const float v = to_f32(row[e]); ss = fmaf(v, v, ss); }
    fq = 1.0f / sqrtf(block_sum(ss, red) / (float)nq + eps);
  }
  if (k_norm_w != nullptr) {
    float ss = 0.f;
    for (int e = tid; e < nk; e += AP_THREADS) {
      const float v = to_f32(row[nq + e]);
      ss = fmaf(v, v, ss);
    }
    fk = 1.0f / sqrtf(block_sum(ss, red) / (float)nk + eps);
  }
  if (temp_coef != 0.f) fq *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every + 1));
  for (int i = tid; i < H * D; i += AP_THREADS) {
    const int h = i / D, e = i % D;
    float v = 0.f;
    if (e < d) v = to_f32(row[h * d + e]) * fq * (q_norm_w ? q_norm_w[h * d + e] : 1.f);
    from_f32(q_out + (size_t)t * H * D + i, v);
  }
  if (k_pool == nullptr) return;
  const size_t page = (size_t)block_tables[(size_t)row_seg[t] * max_blocks + pos / ps];
  const int slot = pos % ps;
  for (int i = tid; i < G * D; i += AP_THREADS) {
    const int g = i / D, e = i % D;
    float kv = 0.f, vv = 0.f;
    if (e < d) kv = to_f32(row[nq + g * d + e]) * fk * (k_norm_w ? k_norm_w[g * d + e] : 1.f);
    if (e < dv) vv = to_f32(row[nq + nk + g * dv + e]);
    from_f32(k_pool + ((page * G + g) * ps + slot) * D + e, kv);
    from_f32(v_pool + ((page * G + g) * D + e) * ps + slot, vv);
  }
}

extern "C" int kappai_projection_norm_store(
    const void* proj, int stride, const float* q_norm_w, const float* k_norm_w, float eps,
    float temp_coef, int temp_every, void* k_pool, void* v_pool, const int* row_pos,
    const int* row_seg, const int* block_tables, int max_blocks, int T, int H, int G, int d,
    int dv, int D, int ps, void* q_out, int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || d < 1 || dv < 1 || D < d || D < dv || ps < 1 || temp_every < 1)
    return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(projection_norm_store_kernel<bf16_t>, dim3(T), dim3(AP_THREADS), 0, stream,
                       (const bf16_t*)proj, stride, q_norm_w, k_norm_w, eps, temp_coef, temp_every,
                       (bf16_t*)k_pool, (bf16_t*)v_pool, row_pos, row_seg, block_tables,
                       max_blocks, H, G, d, dv, D, ps, (bf16_t*)q_out);
  else
    hipLaunchKernelGGL(projection_norm_store_kernel<float>, dim3(T), dim3(AP_THREADS), 0, stream,
                       (const float*)proj, stride, q_norm_w, k_norm_w, eps, temp_coef, temp_every,
                       (float*)k_pool, (float*)v_pool, row_pos, row_seg, block_tables, max_blocks,
                       H, G, d, dv, D, ps, (float*)q_out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// rot_mode 1: pairs (j, j + rot_dims / 2); 2: pairs (2j, 2j + 1).  cos / sin [positions,
// rot_dims / 2].  Only the first rot_dims of the rot places turn; the rest pass as they are.
__device__ __forceinline__ float rotated(const float* x, int e, int rot_dims, int rot_mode,
                                         const float* ct, const float* st) {
  if (e >= rot_dims || rot_mode == 0) return x[e];
  const int half = rot_dims / 2;
  int j, partner;
  bool first;
  if (rot_mode == 1) { first = e < half; j = first ? e : e - half; partner = first ? e + half : e - half; }
  else { first = (e & 1) == 0; j = e / 2; partner = e ^ 1; }
  const float c = ct[j], s = st[j];
  return first ? x[e] * c - x[partner] * s : x[e] * c + x[partner] * s;
}

template <typename T>
__global__ __launch_bounds__(AP_THREADS) void latent_store_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kv, int kv_stride,
    const float* __restrict__ c_norm_w, float eps, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, int rot_dims, int rot_mode, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int d, int rot, int r, int D,
    int ps, T* __restrict__ q_out) {
  extern __shared__ float sh[];            // (H + 1) * rot floats: the parts that turn
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int pos = row_pos[t];
  const T* kvr = kv + (size_t)t * kv_stride;
  const T* qr = q + (size_t)t * q_stride;
  const float* ct = cos_tab + (size_t)pos * (rot_dims / 2);
  const float* st = sin_tab + (size_t)pos * (rot_dims / 2);
  float ss = 0.f;
  for (int e = tid; e < r; e += AP_THREADS) { const float v = to_f32(kvr[e]); ss = fmaf(v, v, ss); }
  for (int i = tid; i < (H + 1) * rot; i += AP_THREADS) {
    const int h = i / rot, e = i % rot;
    sh[i] = h < H ? to_f32(qr[h * (d + rot) + d + e]) : to_f32(kvr[r + e]);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)r + eps);      // (barrier inside)
  for (int i = tid; i < H * (D - r); i += AP_THREADS) {
    const int h = i / (D - r), e = i % (D - r);
    const float v = e < rot ? rotated(sh + h * rot, e, rot_dims, rot_mode, ct, st) : 0.f;
    from_f32(q_out + (size_t)t * H * D + (size_t)h * D + r + e, v);
  }
  if (k_pool == nullptr) return;
  const size_t page = (size_t)block_tables[(size_t)row_seg[t] * max_blocks + pos / ps];
  const int slot = pos % ps;
  for (int e = tid; e < D; e += AP_THREADS) {
    float kvv = 0.f, vv = 0.f;
    if (e < r) kvv = vv = to_f32(kvr[e]) * inv * c_norm_w[e];
    else if (e < r + rot) kvv = rotated(sh + H * rot, e - r, rot_dims, rot_mode, ct, st);
    from_f32(k_pool + (page * ps + slot) * D + e, kvv);
    from_f32(v_pool + (page * D + e) * ps + slot, vv);
  }
}

extern "C" int kappai_latent_store(const void* q, int q_stride, const void* kv, int kv_stride,
                                   const float* c_norm_w, float eps, const float* cos_tab,
                                   const float* sin_tab, int rot_dims, int rot_mode, void* k_pool,
                                   void* v_pool, const int* row_pos, const int* row_seg,
                                   const int* block_tables, int max_blocks, int T, int H, int d,
                                   int rot, int r, int D, int ps, void* q_out, int is_bf16,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || d < 1 || rot < 0 || r < 1 || D < r + rot || rot_dims > rot || rot_dims % 2 ||
      rot_mode < 0 || rot_mode > 2 || (rot_mode && rot_dims && (!cos_tab || !sin_tab)))
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(H + 1) * (rot > 0 ? rot : 1) * sizeof(float);
  if (lds > 48 * 1024) return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(latent_store_kernel<bf16_t>, dim3(T), dim3(AP_THREADS), lds, stream,
                       (const bf16_t*)q, q_stride, (const bf16_t*)kv, kv_stride, c_norm_w, eps,
                       cos_tab, sin_tab, rot_dims, rot_mode, (bf16_t*)k_pool, (bf16_t*)v_pool,
                       row_pos, row_seg, block_tables, max_blocks, H, d, rot, r, D, ps,
                       (bf16_t*)q_out);
  else
    hipLaunchKernelGGL(latent_store_kernel<float>, dim3(T), dim3(AP_THREADS), lds, stream,
                       (const float*)q, q_stride, (const float*)kv, kv_stride, c_norm_w, eps,
                       cos_tab, sin_tab, rot_dims, rot_mode, (float*)k_pool, (float*)v_pool,
                       row_pos, row_seg, block_tables, max_blocks, H, d, rot, r, D, ps,
                       (float*)q_out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// y[t, h, o] = sum_i W[h, o, i] x[t, h, i]: W [H, n_out, n_in] in the activations' dtype, x and y
// with a row stride and a head stride each, float accumulation.  A block takes 32 rows x 64
// outputs of one head; x and W tiles go through LDS in steps of 32 along i.  With `gate` (rows
// of stride g_row, column h n_out + o) the result is multiplied by sigmoid(gate) before it is
// stored.
// ---------------------------------------------------------------------------------------
#define HW_BM 32
#define HW_BN 64
#define HW_BK 32

template <typename T, typename TO>
__global__ __launch_bounds__(256) void headwise_linear_kernel(
    const T* __restrict__ x, int x_row, int x_head, const T* __restrict__ w, int n_out, int n_in,
    TO* __restrict__ y, int y_row, int y_head, int rows, const T* __restrict__ gate, int g_row) {
  __shared__ float xs[HW_BM][HW_BK + 1];
  __shared__ float ws[HW_BN][HW_BK + 1];
  const int h = blockIdx.z, m0 = blockIdx.x * HW_BM, n0 = blockIdx.y * HW_BN;
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;          // outputs 4 tx .. 4 tx + 3, rows 2 ty, 2 ty + 1
  const T* wh = w + (size_t)h * n_out * n_in;
  float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int k0 = 0; k0 < n_in; k0 += HW_BK) {
    for (int i = tid; i < HW_BM * HW_BK; i += 256) {
      const int m = i / HW_BK, k = i % HW_BK;
      xs[m][k] = (m0 + m < rows && k0 + k < n_in)
                     ? to_f32(x[(size_t)(m0 + m) * x_row + (size_t)h * x_head + k0 + k]) : 0.f;
    }
    for (int i = tid; i < HW_BN * HW_BK; i += 256) {
      const int n = i / HW_BK, k = i % HW_BK;
      ws[n][k] = (n0 + n < n_out && k0 + k < n_in) ? to_f32(wh[(size_t)(n0 + n) * n_in + k0 + k])
                                                   : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < HW_BK; ++k) {
      const float a0 = xs[2 * ty][k], a1 = xs[2 * ty + 1][k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = ws[4 * tx + j][k];
        acc[0][j] = fmaf(a0, b, acc[0][j]);
        acc[1][j] = fmaf(a1, b, acc[1][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = m0 + 2 * ty + i;
    if (m >= rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + 4 * tx + j;
      if (n >= n_out) continue;
      float v = acc[i][j];
      if (gate) v /= 1.0f + expf(-to_f32(gate[(size_t)m * g_row + (size_t)h * n_out + n]));
      from_f32(y + (size_t)m * y_row + (size_t)h * y_head + n, v);
    }
  }
}

// The same on the matrix cores, for bfloat16 with n_in, the strides and the pointers multiples of
// eight values.  A wave takes 16 rows x 64 outputs of one head: per step of 32 along i a lane
// loads eight values of its row of x (row lane % 16, values 8 (lane / 16) ..) and of four rows of
// W the same way, and four products W-tile x x-tile^T add up; a lane ends with outputs
// 16 j + 4 (lane / 16) .. + 3 of row lane % 16.  Four waves a block (64 rows); one when there are
// no more than 16 rows.
typedef __attribute__((ext_vector_type(8))) __bf16 hw_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float hw_f32x4_t;

template <typename TO>
__global__ __launch_bounds__(256) void headwise_linear_mfma_kernel(
    const bf16_t* __restrict__ x, int x_row, int x_head, const bf16_t* __restrict__ w, int n_out,
    int n_in, TO* __restrict__ y, int y_row, int y_head, int rows,
    const bf16_t* __restrict__ gate, int g_row) {
  const int h = blockIdx.z, lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int m0 = (blockIdx.x * (blockDim.x / WAVE) + wave) * 16, n0 = blockIdx.y * 64;
  if (m0 >= rows) return;
  const int lr = lane % 16, kq = lane / 16;
  const int m = min(m0 + lr, rows - 1);
  const bf16_t* xr = x + (size_t)m * x_row + (size_t)h * x_head + 8 * kq;
  const bf16_t* wr[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    wr[j] = w + ((size_t)h * n_out + min(n0 + 16 * j + lr, n_out - 1)) * n_in + 8 * kq;
  hw_f32x4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = (hw_f32x4_t){0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  for (int k0 = 0; k0 < n_in; k0 += 32) {
    const bool ok = k0 + 8 * kq < n_in;         // (n_in is a multiple of eight: all or nothing)
    const uint4 xv = ok ? *reinterpret_cast<const uint4*>(xr + k0) : zero;
    uint4 wv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wv[j] = ok ? *reinterpret_cast<const uint4*>(wr[j] + k0) : zero;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(hw_bf16x8_t, wv[j]),
                                                       __builtin_bit_cast(hw_bf16x8_t, xv), acc[j],
                                                       0, 0, 0);
  }
  if (m0 + lr >= rows) return;
  TO* yr = y + (size_t)(m0 + lr) * y_row + (size_t)h * y_head;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int n = n0 + 16 * j + 4 * kq + v;
      if (n >= n_out) continue;
      float r = acc[j][v];
      if (gate)
        r /= 1.0f + expf(-bf16_to_f32(gate[(size_t)(m0 + lr) * g_row + (size_t)h * n_out + n]));
      from_f32(yr + n, r);
    }
}

// out_f32: the results stay float32 although x and W are bfloat16 (what enters a recurrence).
extern "C" int kappai_headwise_linear(const void* x, int x_row, int x_head, const void* w, int H,
                                      int n_out, int n_in, void* y, int y_row, int y_head,
                                      int rows, int is_bf16, int out_f32, const void* gate,
                                      int g_row, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H < 1 || H > 65535 || n_out < 1 || n_in < 1) return (int)hipErrorInvalidValue;
  if (is_bf16 && n_in % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 &&
      ((uintptr_t)x | (uintptr_t)w) % 16 == 0 && (n_out + 63) / 64 <= 65535) {
    const int waves = rows <= 16 ? 1 : 4;
    const dim3 grid((rows + 16 * waves - 1) / (16 * waves), (n_out + 63) / 64, H);
    if (out_f32)
      hipLaunchKernelGGL(headwise_linear_mfma_kernel<float>, grid, dim3(waves * WAVE), 0, stream,
                         (const bf16_t*)x, x_row, x_head, (const bf16_t*)w, n_out, n_in,
                         (float*)y, y_row, y_head, rows, (const bf16_t*)gate, g_row);
    else
      hipLaunchKernelGGL(headwise_linear_mfma_kernel<bf16_t>, grid, dim3(waves * WAVE), 0, stream,
                         (const bf16_t*)x, x_row, x_head, (const bf16_t*)w, n_out, n_in,
                         (bf16_t*)y, y_row, y_head, rows, (const bf16_t*)gate, g_row);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  dim3 grid((rows + HW_BM - 1) / HW_BM, (n_out + HW_BN - 1) / HW_BN, H);
  if (grid.y > 65535) return (int)hipErrorInvalidValue;
  if (is_bf16 && out_f32)
    hipLaunchKernelGGL((headwise_linear_kernel<bf16_t, float>), grid, dim3(256), 0, stream,
                       (const bf16_t*)x, x_row, x_head, (const bf16_t*)w, n_out, n_in, (float*)y,
                       y_row, y_head, rows, (const bf16_t*)gate, g_row);
  else if (is_bf16)
    hipLaunchKernelGGL((headwise_linear_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream,
                       (const bf16_t*)x, x_row, x_head, (const bf16_t*)w, n_out, n_in, (bf16_t*)y,
                       y_row, y_head, rows, (const bf16_t*)gate, g_row);
  else
    hipLaunchKernelGGL((headwise_linear_kernel<float, float>), grid, dim3(256), 0, stream,
                       (const float*)x, x_row, x_head, (const float*)w, n_out, n_in, (float*)y,
                       y_row, y_head, rows, (const float*)gate, g_row);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// rotate_widen_store: grouped-query heads whose queries and keys (d) and values (dv) differ in
// size, with a rotation over the first rot_dims places of every q and k head.  proj [T, H d +
// G d (+ G dv)] as its product left it (biases added).  Queries leave as H heads of D (zeros
// behind d); keys and values go to the pools as G heads of D.  values_are_keys: the projection
// holds no values; a kv head's value is its key as projected, before the rotation (dv = d).
// cos / sin [positions, rot_dims / 2] hold whatever factor the encoding puts on them.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(AP_THREADS) void rotate_widen_store_kernel(
    const T* __restrict__ proj, int stride, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, int rot_dims, int rot_mode, int values_are_keys,
    T* __restrict__ k_pool, T* __restrict__ v_pool, const int* __restrict__ row_pos,
    const int* __restrict__ row_seg, const int* __restrict__ block_tables, int max_blocks, int H,
    int G, int d, int dv, int D, int ps, T* __restrict__ q_out) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const int pos = row_pos[t];
  const T* row = proj + (size_t)t * stride;
  const int nq = H * d, nk = G * d, half = rot_dims / 2;
  const float* ct = cos_tab + (size_t)pos * half;
  const float* st = sin_tab + (size_t)pos * half;
  // place e of the head that starts at `head`: turned by the position, in float32
  auto turned = [&](const T* head, int e) -> float {
    const float x = to_f32(head[e]);
    if (e >= rot_dims || rot_mode == 0) return x;
    int j, partner;
    bool first;
    if (rot_mode == 1) { first = e < half; j = first ? e : e - half; partner = first ? e + half : e - half; }
    else { first = (e & 1) == 0; j = e / 2; partner = e ^ 1; }
    const float y = to_f32(head[partner]), c = ct[j], s = st[j];
    return first ? x * c - y * s : x * c + y * s;
  };
  for (int i = tid; i < H * D; i += AP_THREADS) {
    const int h = i / D, e = i % D;
    from_f32(q_out + (size_t)t * H * D + i, e < d ? turned(row + h * d, e) : 0.f);
  }
  if (k_pool == nullptr) return;
  const size_t page = (size_t)block_tables[(size_t)row_seg[t] * max_blocks + pos / ps];
  const int slot = pos % ps;
  for (int i = tid; i < G * D; i += AP_THREADS) {
    const int g = i / D, e = i % D;
    const T* khead = row + nq + g * d;
    float vv = 0.f;
    if (e < dv) vv = values_are_keys ? to_f32(khead[e]) : to_f32(row[nq + nk + g * dv + e]);
    from_f32(k_pool + ((page * G + g) * ps + slot) * D + e, e < d ? turned(khead, e) : 0.f);
    from_f32(v_pool + ((page * G + g) * D + e) * ps + slot, vv);
  }
}

extern "C" int kappai_rotate_widen_store(
    const void* proj, int stride, const float* cos_tab, const float* sin_tab, int rot_dims,
    int rot_mode, int values_are_keys, void* k_pool, void* v_pool, const int* row_pos,
    const int* row_seg, const int* block_tables, int max_blocks, int T, int H, int G, int d,
    int dv, int D, int ps, void* q_out, int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || d < 1 || dv < 1 || D < d || D < dv || ps < 1 || rot_dims < 0 ||
      rot_dims > d || rot_dims % 2 || rot_mode < 0 || rot_mode > 2 ||
      (values_are_keys && dv != d) || (rot_mode && rot_dims && (!cos_tab || !sin_tab)))
    return (int)hipErrorInvalidValue;
  if (rot_dims == 0) rot_mode = 0;
  if (is_bf16)
    hipLaunchKernelGGL(rotate_widen_store_kernel<bf16_t>, dim3(T), dim3(AP_THREADS), 0, stream,
                       (const bf16_t*)proj, stride, cos_tab, sin_tab, rot_dims, rot_mode,
                       values_are_keys, (bf16_t*)k_pool, (bf16_t*)v_pool, row_pos, row_seg,
                       block_tables, max_blocks, H, G, d, dv, D, ps, (bf16_t*)q_out);
  else
    hipLaunchKernelGGL(rotate_widen_store_kernel<float>, dim3(T), dim3(AP_THREADS), 0, stream,
                       (const float*)proj, stride, cos_tab, sin_tab, rot_dims, rot_mode,
                       values_are_keys, (float*)k_pool, (float*)v_pool, row_pos, row_seg,
                       block_tables, max_blocks, H, G, d, dv, D, ps, (float*)q_out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// head_norm_rotate_store: grouped-query heads whose queries and keys (d) and values (dv) differ
// in size.  Every q and k head is divided by the root mean square of its own d places and
// multiplied by a weight [d] that all heads share (q_norm_w / k_norm_w; null: no norm); then the
// first rot_dims places of the head turn by the row's position.  proj [T, H d + G d + G dv].
// Queries leave as H heads of D (zeros behind d); keys and values go to the pools as G heads of
// D.  A wave a head: the sum of squares stays in the wave; a block takes four heads of a row
// (grid: rows x groups of four heads).
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(AP_THREADS) void head_norm_rotate_store_kernel(
    const T* __restrict__ proj, int stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, int rot_dims, int rot_mode, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int d, int dv, int D,
    int ps, T* __restrict__ q_out) {
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  constexpr int NW = AP_THREADS / WAVE;
  const int pos = row_pos[t];
  const T* row = proj + (size_t)t * stride;
  const int nq = H * d, nk = G * d, half = rot_dims / 2;
  const float* ct = cos_tab + (size_t)pos * half;
  const float* st = sin_tab + (size_t)pos * half;
  size_t page = 0;
  const int slot = pos % ps;
  if (k_pool != nullptr) page = (size_t)block_tables[(size_t)row_seg[t] * max_blocks + pos / ps];
  // heads 0 .. H - 1 are queries, H .. H + G - 1 keys, then the G value heads
  for (int head = blockIdx.y * NW + wave; head < H + 2 * G; head += gridDim.y * NW) {
    if (head >= H + G) {
      if (k_pool == nullptr) continue;
      const int g = head - H - G;
      for (int e = lane; e < D; e += WAVE)
        from_f32(v_pool + ((page * G + g) * D + e) * ps + slot,
                 e < dv ? to_f32(row[nq + nk + g * dv + e]) : 0.f);
      continue;
    }
    const bool is_q = head < H;
    if (!is_q && k_pool == nullptr) continue;
    const T* src = is_q ? row + head * d : row + nq + (head - H) * d;
    const float* w = is_q ? q_norm_w : k_norm_w;
    float r = 1.f;
    if (w != nullptr) {
      float ss = 0.f;
      for (int e = lane; e < d; e += WAVE) { const float v = to_f32(src[e]); ss = fmaf(v, v, ss); }
      r = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
    }
    auto normed = [&](int e) -> float {
      const float v = to_f32(src[e]);
      return w != nullptr ? v * r * w[e] : v;
    };
    T* dst = is_q ? q_out + ((size_t)t * H + head) * D
                  : k_pool + ((page * G + (head - H)) * ps + slot) * D;
    for (int e = lane; e < D; e += WAVE) {
      float v = 0.f;
      if (e < d) {
        v = normed(e);
        if (e < rot_dims && rot_mode != 0) {
          int j, partner;
          bool first;
          if (rot_mode == 1) { first = e < half; j = first ? e : e - half; partner = first ? e + half : e - half; }
          else { first = (e & 1) == 0; j = e / 2; partner = e ^ 1; }
          const float y = normed(partner), c = ct[j], s = st[j];
          v = first ? v * c - y * s : v * c + y * s;
        }
      }
      from_f32(dst + e, v);
    }
  }
}

// The same for bfloat16 heads whose sizes are multiples of eight: a lane takes eight neighbouring
// places of a head (16-byte loads and stores), D / 8 lanes a head (a power of two), several heads
// a wave; sums of squares and rotation partners travel between lanes, not through memory.  The
// rotation pairs place i with i + rot_dims / 2, and rot_dims / 2 is a multiple of eight (or
// nothing turns).
template <int LPH>
__global__ __launch_bounds__(AP_THREADS) void head_norm_rotate_store_vec_kernel(
    const bf16_t* __restrict__ proj, int stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, int rot_dims, bf16_t* __restrict__ k_pool,
    bf16_t* __restrict__ v_pool, const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int d, int dv, int D,
    int ps, bf16_t* __restrict__ q_out) {
  constexpr int HPW = WAVE / LPH, NW = AP_THREADS / WAVE;
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int head = (blockIdx.y * NW + wave) * HPW + lane / LPH, sub = lane % LPH, e0 = sub * 8;
  const int n_heads = H + 2 * G;
  const bool live = head < n_heads && e0 < D && (head < H || k_pool != nullptr);
  const int pos = row_pos[t];
  const bf16_t* row = proj + (size_t)t * stride;
  const int nq = H * d, nk = G * d, half = rot_dims / 2;
  const bool is_v = head >= H + G, is_q = head < H;
  const int width = is_v ? dv : d;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = 0.f;
  if (live && e0 < width) {
    const bf16_t* src = is_q ? row + head * d : is_v ? row + nq + nk + (head - H - G) * dv
                                                     : row + nq + (head - H) * d;
    load8(src + e0, v);
  }
  const float* w = is_q ? q_norm_w : k_norm_w;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss = fmaf(v[i], v[i], ss);
#pragma unroll
  for (int m = 1; m < LPH; m *= 2) ss += __shfl_xor(ss, m);
  if (!is_v && w != nullptr && live && e0 < d) {
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
    float wv[8];
    load8(w + e0, wv);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] *= r * wv[i];
  }
  // rotation partners: the lane half / 8 further on (first half) or back (second half)
  const bool turns = !is_v && rot_dims > 0 && e0 < rot_dims;
  const bool first = e0 < half;
  const int partner = turns ? (first ? lane + half / 8 : lane - half / 8) : lane;
  float pv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) pv[i] = __shfl(v[i], partner);
  if (turns && live) {
    const int j0 = first ? e0 : e0 - half;
    float c[8], sn[8];
    load8(cos_tab + (size_t)pos * half + j0, c);
    load8(sin_tab + (size_t)pos * half + j0, sn);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = first ? v[i] * c[i] - pv[i] * sn[i] : v[i] * c[i] + pv[i] * sn[i];
  }
  if (!live) return;
  if (is_q) {
    store8(q_out + ((size_t)t * H + head) * D + e0, v);
    return;
  }
  const size_t page = (size_t)block_tables[(size_t)row_seg[t] * max_blocks + pos / ps];
  const int slot = pos % ps;
  if (!is_v) {
    store8(k_pool + ((page * G + (head - H)) * ps + slot) * D + e0, v);
  } else {
    bf16_t* dst = v_pool + ((page * G + (head - H - G)) * D + e0) * ps + slot;
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[(size_t)i * ps] = f32_to_bf16(v[i]);
  }
}

extern "C" int kappai_head_norm_rotate_store(
    const void* proj, int stride, const float* q_norm_w, const float* k_norm_w, float eps,
    const float* cos_tab, const float* sin_tab, int rot_dims, int rot_mode, void* k_pool,
    void* v_pool, const int* row_pos, const int* row_seg, const int* block_tables, int max_blocks,
    int T, int H, int G, int d, int dv, int D, int ps, void* q_out, int is_bf16,
    hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || d < 1 || dv < 1 || D < d || D < dv || ps < 1 || rot_dims < 0 ||
      rot_dims > d || rot_dims % 2 || rot_mode < 0 || rot_mode > 2 ||
      (rot_mode && rot_dims && (!cos_tab || !sin_tab)))
    return (int)hipErrorInvalidValue;
  if (rot_dims == 0) rot_mode = 0;
  const int lph = D / 8, half = rot_dims / 2;
  if (is_bf16 && d % 8 == 0 && dv % 8 == 0 && D % 8 == 0 && stride % 8 == 0 &&
      (uintptr_t)proj % 16 == 0 && (uintptr_t)q_out % 16 == 0 && (uintptr_t)k_pool % 16 == 0 &&
      (lph == 1 || lph == 2 || lph == 4 || lph == 8 || lph == 16 || lph == 32) &&
      (rot_mode == 0 || (rot_mode == 1 && half % 8 == 0)) &&
      (!q_norm_w || (uintptr_t)q_norm_w % 16 == 0) && (!k_norm_w || (uintptr_t)k_norm_w % 16 == 0) &&
      (rot_mode == 0 || (((uintptr_t)cos_tab | (uintptr_t)sin_tab) % 16 == 0))) {
    const int per_block = (AP_THREADS / WAVE) * (WAVE / lph);
    const dim3 grid(T, (H + 2 * G + per_block - 1) / per_block);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
#define HNRS_VEC(L)                                                                              \
  hipLaunchKernelGGL(head_norm_rotate_store_vec_kernel<L>, grid, dim3(AP_THREADS), 0, stream,     \
                     (const bf16_t*)proj, stride, q_norm_w, k_norm_w, eps, cos_tab, sin_tab,      \
                     rot_mode ? rot_dims : 0, (bf16_t*)k_pool, (bf16_t*)v_pool, row_pos, row_seg, \
                     block_tables, max_blocks, H, G, d, dv, D, ps, (bf16_t*)q_out)
    switch (lph) {
      case 1: HNRS_VEC(1); break;
      case 2: HNRS_VEC(2); break;
      case 4: HNRS_VEC(4); break;
      case 8: HNRS_VEC(8); break;
      case 16: HNRS_VEC(16); break;
      default: HNRS_VEC(32); break;
    }
#undef HNRS_VEC
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  const dim3 hn_grid(T, min(65535, (H + 2 * G + AP_THREADS / WAVE - 1) / (AP_THREADS / WAVE)));
  if (is_bf16)
    hipLaunchKernelGGL(head_norm_rotate_store_kernel<bf16_t>, hn_grid, dim3(AP_THREADS), 0,
                       stream, (const bf16_t*)proj, stride, q_norm_w, k_norm_w, eps, cos_tab,
                       sin_tab, rot_dims, rot_mode, (bf16_t*)k_pool, (bf16_t*)v_pool, row_pos,
                       row_seg, block_tables, max_blocks, H, G, d, dv, D, ps, (bf16_t*)q_out);
  else
    hipLaunchKernelGGL(head_norm_rotate_store_kernel<float>, hn_grid, dim3(AP_THREADS), 0, stream,
                       (const float*)proj, stride, q_norm_w, k_norm_w, eps, cos_tab, sin_tab,
                       rot_dims, rot_mode, (float*)k_pool, (float*)v_pool, row_pos, row_seg,
                       block_tables, max_blocks, H, G, d, dv, D, ps, (float*)q_out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
