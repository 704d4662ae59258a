// Recurrences with one number of state a channel, S_t = a_t S_(t-1) + b_t, whose a_t and b_t read
// the current token only.  Gates, candidates and the state are float32; the state lives in a slot
// per request [slots, W] and a segment that starts at position 0 starts from zero.
//
// minGRU (KIND 0): a = 1 - z, b = z c with z = sigmoid(pz), c = pu + 1/2 where pu >= 0 and
// sigmoid(pu) below, y_t = S_t * silu(pg).  The projections [T, 3W] = (pz | pu | pg) come with
// their biases added, in float32 or as the bfloat16 a product stored.
//
// Real-gated unit (KIND 1): a = exp(-rate * sigmoid(gr) * sp[c]), b = sqrt(1 - a^2) * sigmoid(gi)
// * u, y_t = S_t * gelu_tanh(py): gr | gi [T, 2W] float32 are the gates before their sigmoid, u
// [T, W] the channel's input (a convolution's result, as stored), py the other branch's projection
// (a view with a row stride, as stored), sp [W] float32 (softplus of the channel's parameter);
// gate_bias [2W] is added to gr | gi before the sigmoid.
#include "common.h"

#define MG_THREADS 256

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ void mingru_gates(float pz, float pu, float& a, float& b) {
  const float z = sigmoid_f(pz);
  const float c = pu >= 0.f ? pu + 0.5f : sigmoid_f(pu);
  a = 1.0f - z;
  b = z * c;
}

// What a scan reads.  KIND 0 uses proj alone.
template <typename TP>
struct scan_in {
  const TP* proj;          // KIND 0: [T, 3W]; KIND 1: the gated branch, rows `y_stride` apart
  const float* gates;      // KIND 1: [T, 2W]: (r | i) for all channels, or with `gate_part` > 0
                           // block by block, (r | i) of `gate_part` channels each
  const float* gate_bias;  // KIND 1: [2W] laid out as a row of gates, added before their sigmoid
  const TP* u;             // KIND 1: [T, W]
  const float* sp;         // KIND 1: [W]
  float rate;              // KIND 1
  int y_stride;            // KIND 1
  int gate_part;           // KIND 1: channels a block of the gates' layout (0: no blocks)
};

// a, b of row t and channel c, and (OUT) the factor on the state that makes the output
template <int KIND, bool OUT, typename TP>
__device__ __forceinline__ void scan_terms(const scan_in<TP>& in, int W, int t, int c, float& a,
                                           float& b, float& g) {
  if (KIND == 0) {
    const TP* p = in.proj + (size_t)t * 3 * W + c;
    mingru_gates(to_f32(p[0]), to_f32(p[W]), a, b);
    if (OUT) {
      const float pg = to_f32(p[2 * W]);
      g = pg * sigmoid_f(pg);
    }
  } else {
    const int part = in.gate_part;
    const int at_r = part ? (c / part) * 2 * part + c % part : c, at_i = at_r + (part ? part : W);
    const float* gp = in.gates + (size_t)t * 2 * W;
    const float uu = to_f32(in.u[(size_t)t * W + c]);
    // (1 - a^2 from the logarithm: a decay close to one loses nothing to cancellation)
    const float la = -in.rate * sigmoid_f(gp[at_r] + in.gate_bias[at_r]) * in.sp[c];
    a = expf(la);
    b = sqrtf(fmaxf(-expm1f(2.0f * la), 0.f)) * sigmoid_f(gp[at_i] + in.gate_bias[at_i]) * uu;
    if (OUT) {
      const float z = to_f32(in.proj[(size_t)t * in.y_stride + c]);
      g = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    }
  }
}

// One thread a (segment, channel), walking the segment's rows in order: what a step of few rows
// a request runs (decoding, short portions).
template <int KIND, typename TP, typename TO>
__global__ __launch_bounds__(MG_THREADS) void mingru_scan_rows_kernel(
    const scan_in<TP> in, float* __restrict__ state, const int* __restrict__ seg_start,
    const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot, int W,
    TO* __restrict__ out) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * MG_THREADS + threadIdx.x;
  if (c >= W) return;
  const int first = seg_start[seg], last = seg_start[seg + 1];
  float* st = state + (size_t)seg_slot[seg] * W + c;
  float S = seg_pos0[seg] > 0 ? *st : 0.f;
  for (int t = first; t < last; ++t) {
    float a, b, g;
    scan_terms<KIND, true>(in, W, t, c, a, b, g);
    S = fmaf(a, S, b);
    from_f32(out + (size_t)t * W + c, S * g);
  }
  *st = S;
}

// Long segments, three passes.  The recurrence S -> a S + b composes: a run of rows acts on the
// state that enters it as S -> A S + B with A the product of its a and B its own result from
// zero.  Pass 1: every chunk of rows of a segment (the host cuts them) gets its (A, B).  Pass 2: a thread a
// (segment, channel) carries the state over the chunks' (A, B) in order and leaves the state at
// every chunk's start in place of them.  Pass 3: every chunk walks its rows from that state and
// writes the outputs.  The state a row sees is the same sum of products whatever the chunks are,
// up to rounding.
template <int KIND, typename TP>
__global__ __launch_bounds__(MG_THREADS) void mingru_chunk_sums_kernel(
    const scan_in<TP> in, const int* __restrict__ chunks, int W,
    float* __restrict__ carry) {
  const int ch = blockIdx.y;
  const int c = blockIdx.x * MG_THREADS + threadIdx.x;
  if (c >= W) return;
  const int first = chunks[3 * ch + 1], n = chunks[3 * ch + 2];
  float A = 1.f, B = 0.f;
  // (four rows' loads at a time, so that they do not wait for one another)
  for (int t0 = first; t0 < first + n; t0 += 4) {
    float a[4], b[4], g;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      scan_terms<KIND, false>(in, W, min(t0 + i, first + n - 1), c, a[i], b[i], g);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (t0 + i >= first + n) break;
      A *= a[i];
      B = fmaf(a[i], B, b[i]);
    }
  }
  carry[((size_t)ch * 3) * W + c] = A;
  carry[((size_t)ch * 3 + 1) * W + c] = B;
}

__global__ __launch_bounds__(MG_THREADS) void mingru_chunk_carry_kernel(
    const int* __restrict__ seg_chunk0, const int* __restrict__ seg_pos0,
    const int* __restrict__ seg_slot, int W, float* __restrict__ carry,
    float* __restrict__ state) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * MG_THREADS + threadIdx.x;
  if (c >= W) return;
  float* st = state + (size_t)seg_slot[seg] * W + c;
  float S = seg_pos0[seg] > 0 ? *st : 0.f;
  const int ch1 = seg_chunk0[seg + 1];
  for (int ch0 = seg_chunk0[seg]; ch0 < ch1; ch0 += 8) {
    float A[8], B[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const size_t ch = (size_t)min(ch0 + i, ch1 - 1);
      A[i] = carry[(ch * 3) * W + c];
      B[i] = carry[(ch * 3 + 1) * W + c];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (ch0 + i >= ch1) break;
      carry[((size_t)(ch0 + i) * 3 + 2) * W + c] = S;      // the state the chunk starts from
      S = fmaf(A[i], S, B[i]);
    }
  }
  *st = S;
}

template <int KIND, typename TP, typename TO>
__global__ __launch_bounds__(MG_THREADS) void mingru_chunk_out_kernel(
    const scan_in<TP> in, const int* __restrict__ chunks, int W,
    const float* __restrict__ carry, TO* __restrict__ out) {
  const int ch = blockIdx.y;
  const int c = blockIdx.x * MG_THREADS + threadIdx.x;
  if (c >= W) return;
  const int first = chunks[3 * ch + 1], n = chunks[3 * ch + 2];
  float S = carry[((size_t)ch * 3 + 2) * W + c];
  for (int t0 = first; t0 < first + n; t0 += 4) {
    float a[4], b[4], g[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      scan_terms<KIND, true>(in, W, min(t0 + i, first + n - 1), c, a[i], b[i], g[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (t0 + i >= first + n) break;
      S = fmaf(a[i], S, b[i]);
      from_f32(out + (size_t)(t0 + i) * W + c, S * g[i]);
    }
  }
}

template <int KIND, typename TP, typename TO>
static void scan_launch(const scan_in<TP>& in, float* state, const int* seg_start,
                        const int* seg_pos0, const int* seg_slot, int S, int W, const int* chunks,
                        const int* seg_chunk0, int n_chunks, float* carry, void* out_v,
                        hipStream_t stream) {
  TO* out = (TO*)out_v;
  const int bx = (W + MG_THREADS - 1) / MG_THREADS;
  if (chunks == nullptr) {
    hipLaunchKernelGGL((mingru_scan_rows_kernel<KIND, TP, TO>), dim3(bx, S), dim3(MG_THREADS), 0,
                       stream, in, state, seg_start, seg_pos0, seg_slot, W, out);
    return;
  }
  hipLaunchKernelGGL((mingru_chunk_sums_kernel<KIND, TP>), dim3(bx, n_chunks), dim3(MG_THREADS), 0,
                     stream, in, chunks, W, carry);
  hipLaunchKernelGGL(mingru_chunk_carry_kernel, dim3(bx, S), dim3(MG_THREADS), 0, stream,
                     seg_chunk0, seg_pos0, seg_slot, W, carry, state);
  hipLaunchKernelGGL((mingru_chunk_out_kernel<KIND, TP, TO>), dim3(bx, n_chunks),
                     dim3(MG_THREADS), 0, stream, in, chunks, W, carry, out);
}

// `chunks` [n_chunks, 3] = (segment, first row, rows) and `seg_chunk0` [S + 1] (first chunk of
// every segment) choose the three-pass form, with `carry` [n_chunks, 3, W] floats of scratch
// (a chunk's A and B, and the state it starts from);
// without them every segment is walked by one thread a channel.
extern "C" int kappai_mingru_scan(const void* proj, int proj_is_bf16, float* state,
                                  const int* seg_start, const int* seg_pos0, const int* seg_slot,
                                  int T, int S, int W, const int* chunks, const int* seg_chunk0,
                                  int n_chunks, float* carry, void* out, int out_is_bf16,
                                  hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (S > 65535 || n_chunks > 65535) return (int)hipErrorInvalidValue;
  if (chunks != nullptr && (n_chunks <= 0 || carry == nullptr || seg_chunk0 == nullptr))
    return (int)hipErrorInvalidValue;
  if (proj_is_bf16 && !out_is_bf16) return (int)hipErrorInvalidValue;
  if (proj_is_bf16)
    scan_launch<0, bf16_t, bf16_t>(scan_in<bf16_t>{(const bf16_t*)proj, nullptr, nullptr, nullptr, nullptr,
                                                   0.f, 0, 0},
                                   state, seg_start, seg_pos0, seg_slot, S, W, chunks, seg_chunk0,
                                   n_chunks, carry, out, stream);
  else if (out_is_bf16)
    scan_launch<0, float, bf16_t>(scan_in<float>{(const float*)proj, nullptr, nullptr, nullptr, nullptr,
                                                 0.f, 0, 0},
                                  state, seg_start, seg_pos0, seg_slot, S, W, chunks, seg_chunk0,
                                  n_chunks, carry, out, stream);
  else
    scan_launch<0, float, float>(scan_in<float>{(const float*)proj, nullptr, nullptr, nullptr, nullptr,
                                                0.f, 0, 0},
                                 state, seg_start, seg_pos0, seg_slot, S, W, chunks, seg_chunk0,
                                 n_chunks, carry, out, stream);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// The real-gated unit through the same kernels; `out` is stored as `u` and `y` are.
extern "C" int kappai_gated_unit_scan(const float* gates, const float* gate_bias, const void* u,
                                      const void* y,
                                      int y_stride, const float* sp, float rate, int gate_part,
                                      int is_bf16,
                                      float* state, const int* seg_start, const int* seg_pos0,
                                      const int* seg_slot, int T, int S, int W, const int* chunks,
                                      const int* seg_chunk0, int n_chunks, float* carry, void* out,
                                      hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (S > 65535 || n_chunks > 65535 || W < 1 || y_stride < W || gate_bias == nullptr ||
      gate_part < 0 || (gate_part && W % gate_part))
    return (int)hipErrorInvalidValue;
  if (chunks != nullptr && (n_chunks <= 0 || carry == nullptr || seg_chunk0 == nullptr))
    return (int)hipErrorInvalidValue;
  if (is_bf16)
    scan_launch<1, bf16_t, bf16_t>(scan_in<bf16_t>{(const bf16_t*)y, gates, gate_bias, (const bf16_t*)u, sp,
                                                   rate, y_stride, gate_part},
                                   state, seg_start, seg_pos0, seg_slot, S, W, chunks, seg_chunk0,
                                   n_chunks, carry, out, stream);
  else
    scan_launch<1, float, float>(scan_in<float>{(const float*)y, gates, gate_bias, (const float*)u, sp, rate,
                                                y_stride, gate_part},
                                 state, seg_start, seg_pos0, seg_slot, S, W, chunks, seg_chunk0,
                                 n_chunks, carry, out, stream);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// A decode step of the real-gated unit in one kernel, for steps whose every segment is a single
// row: the convolution over the request's history (and the history brought up to date), both
// gates of a block, the recurrence and the gated output.  A block of threads takes a (row, block
// of channels): u of the block's `part` channels is made and kept in LDS (rounded as the
// convolution's own kernel stores it), a thread takes a row of the block's gate matrix (W [blocks,
// 2 part, part]: the rows of r, then those of i), and a thread a channel finishes.
//   proj [T, >= 2W] rows `stride` apart: (x | y) with biases added; taps [W, n], conv_bias [W],
//   conv_state [slots, n - 1, W] oldest first; gate_bias [blocks, 2 part]; sp [W] = softplus(lam);
//   state [slots, W]; seg_pos0 / seg_slot [T]; out [T, W] stored as proj is.
// ---------------------------------------------------------------------------------------
#define GU_STEP_THREADS 256
__device__ __forceinline__ void gu_load8(const float* p, float (&w)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
}
__device__ __forceinline__ void gu_load8(const bf16_t* p, float (&w)[8]) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  const unsigned v[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    w[2 * k] = __uint_as_float(v[k] << 16);
    w[2 * k + 1] = __uint_as_float(v[k] & 0xffff0000u);
  }
}

template <typename TP>
__global__ __launch_bounds__(GU_STEP_THREADS) void gated_unit_step_kernel(
    const TP* __restrict__ proj, int stride, const float* __restrict__ taps, int n_taps,
    const float* __restrict__ conv_bias, float* __restrict__ conv_state,
    const TP* __restrict__ gate_w, const float* __restrict__ gate_bias,
    const float* __restrict__ sp, float rate, float* __restrict__ state,
    const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot, int W, int part,
    TP* __restrict__ out) {
  extern __shared__ float gu_lds[];
  float* us = gu_lds;                 // [part]
  float* gs = gu_lds + part;          // [2 part]
  const int t = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int pos = seg_pos0[t], slot = seg_slot[t], keep = n_taps - 1;
  const TP* row = proj + (size_t)t * stride;
  float* hist = conv_state + (size_t)slot * keep * W;
  for (int i = tid; i < part; i += GU_STEP_THREADS) {
    const int c = b * part + i;
    const float x = to_f32(row[c]);
    const float* tp = taps + (size_t)c * n_taps;
    float acc = tp[keep] * x;
    float older[16];
    for (int j = 0; j < keep; ++j) {
      // entry j of the history is the token `keep - j` before this one
      older[j] = keep - j <= pos ? hist[(size_t)j * W + c] : 0.f;
      acc = fmaf(tp[j], older[j], acc);
    }
    for (int j = 0; j + 1 < keep; ++j) hist[(size_t)j * W + c] = older[j + 1];
    if (keep > 0) hist[(size_t)(keep - 1) * W + c] = x;
    TP stored;
    from_f32(&stored, acc + conv_bias[c]);
    us[i] = to_f32(stored);
  }
  __syncthreads();
  // a thread a row of the block's gate matrix: its loads do not wait for one another, and the
  // block's u is read from LDS by all lanes at once
  const TP* wb = gate_w + (size_t)b * 2 * part * part;
  for (int o = tid; o < 2 * part; o += GU_STEP_THREADS) {
    const TP* wr = wb + (size_t)o * part;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    int i = 0;
    if (part % 8 == 0 && ((uintptr_t)wb % 16) == 0) {
      for (; i < part; i += 8) {
        float w[8];
        gu_load8(wr + i, w);
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[k % 4] = fmaf(w[k], us[i + k], acc[k % 4]);
      }
    }
    for (; i < part; ++i) acc[0] = fmaf(to_f32(wr[i]), us[i], acc[0]);
    gs[o] = (acc[0] + acc[1]) + (acc[2] + acc[3]) + gate_bias[(size_t)b * 2 * part + o];
  }
  __syncthreads();
  for (int i = tid; i < part; i += GU_STEP_THREADS) {
    const int c = b * part + i;
    const float la = -rate * sigmoid_f(gs[i]) * sp[c];
    const float a = expf(la);
    const float in = sqrtf(fmaxf(-expm1f(2.0f * la), 0.f)) * sigmoid_f(gs[part + i]) * us[i];
    float* st = state + (size_t)slot * W + c;
    const float S = fmaf(a, pos > 0 ? *st : 0.f, in);
    *st = S;
    const float z = to_f32(row[W + c]);
    const float g = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    from_f32(out + (size_t)t * W + c, S * g);
  }
}

extern "C" int kappai_gated_unit_step(const void* proj, int stride, const float* taps, int n_taps,
                                      const float* conv_bias, float* conv_state,
                                      const void* gate_w, const float* gate_bias, const float* sp,
                                      float rate, float* state, const int* seg_pos0,
                                      const int* seg_slot, int T, int W, int blocks, int is_bf16,
                                      void* out, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W < 1 || blocks < 1 || blocks > 65535 || W % blocks || n_taps < 1 || n_taps > 17 ||
      stride < 2 * W || W / blocks > 4096 || !conv_bias || !gate_bias || !sp ||
      (n_taps > 1 && !conv_state))
    return (int)hipErrorInvalidValue;
  const int part = W / blocks;
  const size_t lds = (size_t)3 * part * sizeof(float);
  const dim3 grid(T, blocks);
  if (is_bf16)
    hipLaunchKernelGGL(gated_unit_step_kernel<bf16_t>, grid, dim3(GU_STEP_THREADS), lds, stream,
                       (const bf16_t*)proj, stride, taps, n_taps, conv_bias, conv_state,
                       (const bf16_t*)gate_w, gate_bias, sp, rate, state, seg_pos0, seg_slot, W,
                       part, (bf16_t*)out);
  else
    hipLaunchKernelGGL(gated_unit_step_kernel<float>, grid, dim3(GU_STEP_THREADS), lds, stream,
                       (const float*)proj, stride, taps, n_taps, conv_bias, conv_state,
                       (const float*)gate_w, gate_bias, sp, rate, state, seg_pos0, seg_slot, W,
                       part, (float*)out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
