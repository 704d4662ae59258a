// Recurrences whose state is a matrix per head, S [d, dv] in float32 (a slot per request; kept
// column by column, [dv, d]), with a
// decay per key channel:
//   gated linear attention   S <- diag(a) S + k v^T                      o = S^T q
//   gated delta rule         S <- diag(a) S; u = beta (v - S^T k); S <- S + k u^T;  o = S^T q
//   bonus for the own token  o = (S + diag(u) k v^T)^T q;  S <- diag(a) S + k v^T   (the read-out
//                            sees the state before the token and the token itself times u [H, d])
// and what stands around them: the short causal convolution with SiLU on the projections, the
// decays / unit vectors / step sizes in float32, and the per-head RMS norm with its gate.
//
// A column of S (one value channel) never meets another column, so the work of a (segment, head)
// is spread over lanes by value channel, and a column's d rows over KS neighbouring lanes whose
// partial dot products meet by lane exchanges.  Tokens of a segment are walked in order; a
// segment that starts at position 0 starts from zero, whatever the slot holds.
#include "common.h"

#define LA_THREADS 256

__device__ __forceinline__ float la_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float la_softplus(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

// ---------------------------------------------------------------------------------------
// Short causal convolution per channel, then SiLU (act 1) or nothing (act 0), with an optional
// bias [C] added before the activation.  x [T, >= C] with a row stride, taps [C, n]
// (the last column meets the current token), state [slots, n - 1, C] float32: the last n - 1
// inputs of the request, oldest first.  One thread a (row, channel) for the outputs; a second
// kernel rewrites the state after the outputs are made.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(LA_THREADS) void conv_silu_kernel(
    const T* __restrict__ x, int x_stride, const float* __restrict__ taps, int n_taps,
    const float* __restrict__ state, const int* __restrict__ row_pos,
    const int* __restrict__ row_seg, const int* __restrict__ seg_start,
    const int* __restrict__ seg_slot, int C, const float* __restrict__ bias, int act,
    T* __restrict__ out) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * LA_THREADS + threadIdx.x;
  if (c >= C) return;
  // The sum over the rows before this one as if all of them were the segment's own: these loads
  // wait for no table, so they are on their way while the row's segment, its start and its slot
  // are read one after the other.  Only the first rows of a segment take the other path.
  float ahead = 0.f;
  for (int j = 0; j < n_taps; ++j) {
    const int tt = t - (n_taps - 1 - j);
    if (tt >= 0) ahead = fmaf(taps[(size_t)c * n_taps + j], to_f32(x[(size_t)tt * x_stride + c]), ahead);
  }
  const int seg = row_seg[t], first = seg_start[seg];
  float acc = 0.f;
  if (t - (n_taps - 1) >= first) {
    acc = ahead;
  } else {
    const int pos = row_pos[t];
    const float* st = state + (size_t)seg_slot[seg] * (n_taps - 1) * C;
    for (int j = 0; j < n_taps; ++j) {
      const int back = n_taps - 1 - j;          // how many tokens before this one
      if (back > pos) continue;                 // before the start of the sequence: zero
      float v;
      if (t - back >= first) v = to_f32(x[(size_t)(t - back) * x_stride + c]);
      else v = st[(size_t)(n_taps - 1 - (back - (t - first))) * C + c];
      acc = fmaf(taps[(size_t)c * n_taps + j], v, acc);
    }
  }
  if (bias != nullptr) acc += bias[c];
  from_f32(out + (size_t)t * C + c, act ? acc * la_sigmoid(acc) : acc);
}

template <typename T>
__global__ __launch_bounds__(LA_THREADS) void conv_state_kernel(
    const T* __restrict__ x, int x_stride, int n_taps, float* __restrict__ state,
    const int* __restrict__ seg_start, const int* __restrict__ seg_pos0,
    const int* __restrict__ seg_slot, int C) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * LA_THREADS + threadIdx.x;
  if (c >= C) return;
  const int first = seg_start[seg], n = seg_start[seg + 1] - first, keep = n_taps - 1;
  float* st = state + (size_t)seg_slot[seg] * keep * C + c;
  const bool fresh = seg_pos0[seg] == 0;
  // entry i of the new history is input number n - keep + i of the segment; a negative number
  // reaches back into the old history (zero for a request that has just begun)
  float kept[16];
  for (int i = 0; i < keep; ++i) {
    const int src = n - keep + i;
    if (src >= 0) kept[i] = to_f32(x[(size_t)(first + src) * x_stride + c]);
    else kept[i] = fresh ? 0.f : st[(size_t)(keep + src) * C];
  }
  for (int i = 0; i < keep; ++i) st[(size_t)i * C] = kept[i];
}

extern "C" int kappai_conv_silu(const void* x, int x_stride, const float* taps, int n_taps,
                                float* state, const int* row_pos, const int* row_seg,
                                const int* seg_start, const int* seg_pos0, const int* seg_slot,
                                int T, int S, int C, const float* bias, int act, void* out,
                                int is_bf16, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (n_taps < 1 || n_taps > 17 || S > 65535 || C > 65535 * LA_THREADS) return (int)hipErrorInvalidValue;
  const int bx = (C + LA_THREADS - 1) / LA_THREADS;
  if (is_bf16) {
    hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, dim3(T, bx), dim3(LA_THREADS), 0, stream,
                       (const bf16_t*)x, x_stride, taps, n_taps, state, row_pos, row_seg,
                       seg_start, seg_slot, C, bias, act, (bf16_t*)out);
    if (n_taps > 1)
      hipLaunchKernelGGL(conv_state_kernel<bf16_t>, dim3(bx, S), dim3(LA_THREADS), 0, stream,
                         (const bf16_t*)x, x_stride, n_taps, state, seg_start, seg_pos0, seg_slot,
                         C);
  } else {
    hipLaunchKernelGGL(conv_silu_kernel<float>, dim3(T, bx), dim3(LA_THREADS), 0, stream,
                       (const float*)x, x_stride, taps, n_taps, state, row_pos, row_seg, seg_start,
                       seg_slot, C, bias, act, (float*)out);
    if (n_taps > 1)
      hipLaunchKernelGGL(conv_state_kernel<float>, dim3(bx, S), dim3(LA_THREADS), 0, stream,
                         (const float*)x, x_stride, n_taps, state, seg_start, seg_pos0, seg_slot,
                         C);
  }
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// Token shift: with h' the row before (the request's last row of the step before for a segment's
// first row: state [slots, W] float32; zeros at position 0), out[m] = h + (h' - h) * mu[m] for
// each of the n_mix rows of mu [n_mix, W], out [n_mix, T, W].  A thread a (row, channel); a
// second kernel leaves every segment's last row as its state after the outputs are made.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(LA_THREADS) void token_shift_mix_kernel(
    const T* __restrict__ h, int h_stride, const float* __restrict__ mu, int n_mix,
    const float* __restrict__ state, const int* __restrict__ row_pos,
    const int* __restrict__ row_seg, const int* __restrict__ seg_start,
    const int* __restrict__ seg_slot, int rows, int W, T* __restrict__ out) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * LA_THREADS + threadIdx.x;
  if (c >= W) return;
  const int seg = row_seg[t];
  const float cur = to_f32(h[(size_t)t * h_stride + c]);
  float before = 0.f;
  if (row_pos[t] > 0)
    before = t > seg_start[seg] ? to_f32(h[(size_t)(t - 1) * h_stride + c])
                                : state[(size_t)seg_slot[seg] * W + c];
  const float diff = before - cur;
  for (int m = 0; m < n_mix; ++m)
    from_f32(out + ((size_t)m * rows + t) * W + c, fmaf(diff, mu[(size_t)m * W + c], cur));
}

template <typename T>
__global__ __launch_bounds__(LA_THREADS) void token_shift_state_kernel(
    const T* __restrict__ h, int h_stride, float* __restrict__ state,
    const int* __restrict__ seg_start, const int* __restrict__ seg_slot, int W) {
  const int seg = blockIdx.y;
  const int c = blockIdx.x * LA_THREADS + threadIdx.x;
  if (c >= W) return;
  const int last = seg_start[seg + 1] - 1;
  if (last < seg_start[seg]) return;
  state[(size_t)seg_slot[seg] * W + c] = to_f32(h[(size_t)last * h_stride + c]);
}

extern "C" int kappai_token_shift_mix(const void* h, int h_stride, const float* mu, int n_mix,
                                      float* state, const int* row_pos, const int* row_seg,
                                      const int* seg_start, const int* seg_slot, int T, int S,
                                      int W, void* out, int is_bf16, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (n_mix < 1 || W < 1 || S > 65535 || W > 65535 * LA_THREADS) return (int)hipErrorInvalidValue;
  const int bx = (W + LA_THREADS - 1) / LA_THREADS;
  if (is_bf16) {
    hipLaunchKernelGGL(token_shift_mix_kernel<bf16_t>, dim3(T, bx), dim3(LA_THREADS), 0, stream,
                       (const bf16_t*)h, h_stride, mu, n_mix, state, row_pos, row_seg, seg_start,
                       seg_slot, T, W, (bf16_t*)out);
    hipLaunchKernelGGL(token_shift_state_kernel<bf16_t>, dim3(bx, S), dim3(LA_THREADS), 0, stream,
                       (const bf16_t*)h, h_stride, state, seg_start, seg_slot, W);
  } else {
    hipLaunchKernelGGL(token_shift_mix_kernel<float>, dim3(T, bx), dim3(LA_THREADS), 0, stream,
                       (const float*)h, h_stride, mu, n_mix, state, row_pos, row_seg, seg_start,
                       seg_slot, T, W, (float*)out);
    hipLaunchKernelGGL(token_shift_state_kernel<float>, dim3(bx, S), dim3(LA_THREADS), 0, stream,
                       (const float*)h, h_stride, state, seg_start, seg_slot, W);
  }
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// What enters the recurrence, in float32: a wave a (row, head).
//   qf, kf [T, Hk, d]   q and k (head h reads q/k head h / (H / Hk)), optionally made unit
//                       vectors x / sqrt(sum x^2 + unit_eps); q also times q_scale
//                       (act: silu of the projection as it is stored, rounded as it is stored)
//   af [T, H, d]        the decay, by decay_kind: 0  exp(-rate[h] * softplus(sign * (z + z_bias)))
//                                                 1  exp(-exp(z + z_bias))
//                                                 2  rate[h] itself (z is not read)
//   bf [T, H]           sigmoid(b) when b is given
//   vf [T, H, dv]       silu(v), rounded as v is stored, when v is given
// ---------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float la_stored_silu(float x) {
  T r;
  from_f32(&r, x * la_sigmoid(x));
  return to_f32(r);
}

template <typename T>
__global__ __launch_bounds__(WAVE) void recurrence_prep_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k, int k_stride,
    const T* __restrict__ z, int z_stride, const float* __restrict__ z_bias,
    const float* __restrict__ rate, float sign, const T* __restrict__ b, int b_stride, int H,
    int Hk, int d, int unit, float unit_eps, float q_scale, int act, int decay_kind,
    const T* __restrict__ v, int v_stride, int dv, float* __restrict__ qf,
    float* __restrict__ kf, float* __restrict__ af, float* __restrict__ bf,
    float* __restrict__ vf) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  if (v != nullptr) {
    const T* vr = v + (size_t)t * v_stride + (size_t)h * dv;
    for (int e = lane; e < dv; e += WAVE)
      vf[((size_t)t * H + h) * dv + e] = la_stored_silu<T>(to_f32(vr[e]));
  }
  if (h < Hk && act) {
    const T* qr = q + (size_t)t * q_stride + (size_t)h * d;
    const T* kr = k + (size_t)t * k_stride + (size_t)h * d;
    for (int e = lane; e < d; e += WAVE) {
      qf[((size_t)t * Hk + h) * d + e] = la_stored_silu<T>(to_f32(qr[e])) * q_scale;
      kf[((size_t)t * Hk + h) * d + e] = la_stored_silu<T>(to_f32(kr[e]));
    }
  } else if (h < Hk) {
    const T* qr = q + (size_t)t * q_stride + (size_t)h * d;
    const T* kr = k + (size_t)t * k_stride + (size_t)h * d;
    float sq = 0.f, sk = 0.f;
    for (int e = lane; e < d; e += WAVE) {
      const float a = to_f32(qr[e]), c = to_f32(kr[e]);
      sq = fmaf(a, a, sq);
      sk = fmaf(c, c, sk);
    }
    float fq = q_scale, fk = 1.f;
    if (unit) {
      fq = q_scale / sqrtf(wave_sum(sq) + unit_eps);
      fk = 1.0f / sqrtf(wave_sum(sk) + unit_eps);
    }
    for (int e = lane; e < d; e += WAVE) {
      qf[((size_t)t * Hk + h) * d + e] = to_f32(qr[e]) * fq;
      kf[((size_t)t * Hk + h) * d + e] = to_f32(kr[e]) * fk;
    }
  }
  const float r = rate != nullptr ? rate[h] : 1.f;
  if (decay_kind == 2) {
    for (int e = lane; e < d; e += WAVE) af[((size_t)t * H + h) * d + e] = r;
  } else {
    const T* zr = z + (size_t)t * z_stride + (size_t)h * d;
    for (int e = lane; e < d; e += WAVE) {
      const float zz = to_f32(zr[e]) + (z_bias ? z_bias[(size_t)h * d + e] : 0.f);
      af[((size_t)t * H + h) * d + e] =
          decay_kind == 1 ? expf(-expf(zz)) : expf(-r * la_softplus(sign * zz));
    }
  }
  if (b != nullptr && lane == 0)
    bf[(size_t)t * H + h] = la_sigmoid(to_f32(b[(size_t)t * b_stride + h]));
}

extern "C" int kappai_recurrence_prep(const void* q, int q_stride, const void* k, int k_stride,
                                      const void* z, int z_stride, const float* z_bias,
                                      const float* rate, float sign, const void* b, int b_stride,
                                      int T, int H, int Hk, int d, int unit, float unit_eps,
                                      float q_scale, int act, int decay_kind, const void* v,
                                      int v_stride, int dv, float* qf, float* kf, float* af,
                                      float* bf, float* vf, int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || Hk < 1 || H % Hk || H > 65535 || d < 1 || decay_kind < 0 || decay_kind > 2 ||
      (decay_kind != 2 && z == nullptr) || (decay_kind != 1 && rate == nullptr) ||
      (act && unit) || (v != nullptr && (vf == nullptr || dv < 1)))
    return (int)hipErrorInvalidValue;
  if (is_bf16)
    hipLaunchKernelGGL(recurrence_prep_kernel<bf16_t>, dim3(T, H), dim3(WAVE), 0, stream,
                       (const bf16_t*)q, q_stride, (const bf16_t*)k, k_stride, (const bf16_t*)z,
                       z_stride, z_bias, rate, sign, (const bf16_t*)b, b_stride, H, Hk, d, unit,
                       unit_eps, q_scale, act, decay_kind, (const bf16_t*)v, v_stride, dv, qf, kf,
                       af, bf, vf);
  else
    hipLaunchKernelGGL(recurrence_prep_kernel<float>, dim3(T, H), dim3(WAVE), 0, stream,
                       (const float*)q, q_stride, (const float*)k, k_stride, (const float*)z,
                       z_stride, z_bias, rate, sign, (const float*)b, b_stride, H, Hk, d, unit,
                       unit_eps, q_scale, act, decay_kind, (const float*)v, v_stride, dv, qf, kf,
                       af, bf, vf);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// The recurrence itself.  Lane (c, s) of a wave keeps R rows of column c of S in registers (eight;
// sixteen for key sizes beyond 512), in groups of four: rows 4 (j KS + s) .. + 3 for j = 0 ..
// R / 4 - 1, so that the KS lanes of a column read neighbouring 16-byte pieces of q, k and the
// decay (no two on one LDS bank).  Few rows a lane, because a wave alone on its SIMD issues an
// instruction only every ten cycles or so: the walk along the tokens is as fast as a wave's
// instructions per token are few, and idle SIMDs are there to take more waves.  These lanes
// are neighbours, and their partial dot products meet by data-parallel moves.  MODE 0: the plain gated sum; 1: the delta rule (needs beta); 2: the bonus for the own token.
// In memory a head's matrix lies column by column: state [slots, H, dv, d], so that a lane's rows
// are consecutive and a wave's columns one stretch.
//
// Two kernels.  The block form: up to four waves share the q, k and decay rows of their head
// (two when the grid would not fill the chip otherwise: what a CU's waves read from LDS per token
// bounds the walk, so a long prompt's waves are spread over more CUs).
// The tokens of a segment come in chunks of `tb`: while a chunk is worked on out of LDS, every
// thread already holds its share of the next chunk's loads in registers, so the walk along the
// tokens never waits for global memory.  The wave form reads each token from global memory one
// ahead; it serves the shapes whose rows do not fit the block form's registers.
// ---------------------------------------------------------------------------------------
#define LA_MAX_WAVES 4
#define LA_MAX_CHUNK 16

// the r-th of a lane's rows
template <int KS>
__device__ __forceinline__ int la_row(int s, int r) { return 4 * ((r / 4) * KS + s) + r % 4; }

template <int KS>
__device__ __forceinline__ float ks_sum(float v) {
  if (KS >= 2) v += dpp_move<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  if (KS >= 4) v += dpp_move<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  if (KS >= 8) v += dpp_move<0x141>(v);     // the other quad of a half row (row_half_mirror)
  if (KS >= 16) v += dpp_move<0x140>(v);    // the other half of a row (row_mirror)
  if (KS >= 32) v += lane_xor16(v);
  if (KS >= 64) v += lane_xor32(v);
  return v;
}

template <int KS, int R>
__device__ __forceinline__ void la_load_rows(const float* __restrict__ st, int s, int d,
                                             bool carry, float (&S)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = 0.f;
  if (!carry) return;
  if (d % 4 == 0) {
#pragma unroll
    for (int r4 = 0; r4 < R; r4 += 4) {
      const int row = la_row<KS>(s, r4);
      if (row < d) {
        const float4 x = *reinterpret_cast<const float4*>(st + row);
        S[r4] = x.x; S[r4 + 1] = x.y; S[r4 + 2] = x.z; S[r4 + 3] = x.w;
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (la_row<KS>(s, r) < d) S[r] = st[la_row<KS>(s, r)];
  }
}

template <int KS, int R>
__device__ __forceinline__ void la_store_rows(float* __restrict__ st, int s, int d,
                                              const float (&S)[R]) {
  if (d % 4 == 0) {
#pragma unroll
    for (int r4 = 0; r4 < R; r4 += 4) {
      const int row = la_row<KS>(s, r4);
      if (row < d)
        *reinterpret_cast<float4*>(st + row) =
            make_float4(S[r4], S[r4 + 1], S[r4 + 2], S[r4 + 3]);
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (la_row<KS>(s, r) < d) st[la_row<KS>(s, r)] = S[r];
  }
}

// One token: S, the lane's rows of q, k and the decay, the column's v, the head's beta.  The dot
// products are summed in four strands (rows r, r + 4, ...) that meet at the end: four short
// chains of dependent operations instead of one long one.
template <int KS, int R, int MODE>
__device__ __forceinline__ float la_token(float (&S)[R], const float (&qc)[R],
                                          const float (&kc)[R], const float (&ac)[R],
                                          const float (&uc)[R], float vc, float bc) {
  float o[4] = {0.f, 0.f, 0.f, 0.f};
  if (MODE == 2) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float kv = kc[r] * vc;
      o[r % 4] = fmaf(fmaf(uc[r], kv, S[r]), qc[r], o[r % 4]);
      S[r] = fmaf(ac[r], S[r], kv);
    }
  } else if (MODE == 1) {
    float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] *= ac[r];
      dot[r % 4] = fmaf(S[r], kc[r], dot[r % 4]);
    }
    const float u = bc * (vc - ks_sum<KS>((dot[0] + dot[1]) + (dot[2] + dot[3])));
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] = fmaf(kc[r], u, S[r]);
      o[r % 4] = fmaf(S[r], qc[r], o[r % 4]);
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] = fmaf(ac[r], S[r], kc[r] * vc);
      o[r % 4] = fmaf(S[r], qc[r], o[r % 4]);
    }
  }
  return ks_sum<KS>((o[0] + o[1]) + (o[2] + o[3]));
}

// LDS, per token of a chunk: q [dp], k [dp], a [dp] (dp = KS * R, zeros beyond d), v [NWC], beta,
// padded to `rec` floats (a multiple of four).  d is a multiple of four and NWC a power of two
// (1 << nwc_log2).  A thread's places in a chunk are fixed: LA_QS 16-byte pieces of each of q, k
// and the decay (piece i = tid + j * threads: token i / (d / 4), floats 4 (i % (d / 4)) ..), and
// up to LA_MAX_CHUNK values of v.
#define LA_QS 4
template <int KS, int R, int MODE, typename TV>
__global__ __launch_bounds__(LA_MAX_WAVES * WAVE) void matrix_state_scan_block_kernel(
    const float* __restrict__ qf, const float* __restrict__ kf, const float* __restrict__ af,
    const float* __restrict__ bf, const TV* __restrict__ v, int v_stride,
    float* __restrict__ state, const int* __restrict__ seg_start,
    const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot, int H, int Hk, int d,
    int dv, int tb, int rec, int nwc_log2, float* __restrict__ out) {
  extern __shared__ float sh_scan[];
  constexpr int COLS = WAVE / KS;
  constexpr int DP = KS * R;
  const int nthr = blockDim.x, tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int NWC = 1 << nwc_log2;
  const int seg = blockIdx.z, h = blockIdx.y, c0 = blockIdx.x * NWC;
  const int s = lane % KS, cl = wave * COLS + lane / KS, c = c0 + cl;
  const bool col_ok = c < dv;
  const int cc = col_ok ? c : dv - 1;
  const int hk = h / (H / Hk);
  const int first = seg_start[seg], last = seg_start[seg + 1];
  float* st = state + (((size_t)seg_slot[seg] * H + h) * dv + cc) * d;
  float S[R];
  la_load_rows<KS, R>(st, s, d, seg_pos0[seg] > 0, S);
  float uc[R];      // MODE 2: the lane's rows of the head's bonus, which `bf` then holds [H, d]
#pragma unroll
  for (int r = 0; r < R; ++r)
    uc[r] = MODE == 2 && la_row<KS>(s, r) < d ? bf[(size_t)h * d + la_row<KS>(s, r)] : 0.f;

  // the thread's places
  const int g4 = d / 4;
  int p_tok[LA_QS], p_qk[LA_QS], p_a[LA_QS], p_lds[LA_QS];
#pragma unroll
  for (int j = 0; j < LA_QS; ++j) {
    const int i = tid + j * nthr, tt = i / g4, g = i - tt * g4;
    p_tok[j] = tt;
    p_qk[j] = (tt * Hk + hk) * d + 4 * g;
    p_a[j] = (tt * H + h) * d + 4 * g;
    p_lds[j] = tt * rec + 4 * g;
  }
  const int v_slots = (tb * NWC + nthr - 1) / nthr;
  const int v_col = min(c0 + (tid & (NWC - 1)), dv - 1);
  float4 sq[LA_QS], sk[LA_QS], sa[LA_QS];
  float sv[LA_MAX_CHUNK], sb = 0.f;
  // the thread's share of the chunk that starts at token t0 (n tokens), into registers ...
  auto fetch = [&](int t0, int n) {
    const float* qb = qf + (size_t)t0 * Hk * d;
    const float* kb = kf + (size_t)t0 * Hk * d;
    const float* ab = af + (size_t)t0 * H * d;
#pragma unroll
    for (int j = 0; j < LA_QS; ++j)
      if (p_tok[j] < n) {
        sq[j] = *reinterpret_cast<const float4*>(qb + p_qk[j]);
        sk[j] = *reinterpret_cast<const float4*>(kb + p_qk[j]);
        sa[j] = *reinterpret_cast<const float4*>(ab + p_a[j]);
      }
#pragma unroll
    for (int j = 0; j < LA_MAX_CHUNK; ++j)
      if (j < v_slots) {
        const int tt = (tid + j * nthr) >> nwc_log2;
        if (tt < n) sv[j] = to_f32(v[(size_t)(t0 + tt) * v_stride + (size_t)h * dv + v_col]);
      }
    if (MODE == 1 && tid < n) sb = bf[(size_t)(t0 + tid) * H + h];
  };
  // ... and from the registers to LDS
  auto put = [&](int n) {
#pragma unroll
    for (int j = 0; j < LA_QS; ++j)
      if (p_tok[j] < n) {
        *reinterpret_cast<float4*>(sh_scan + p_lds[j]) = sq[j];
        *reinterpret_cast<float4*>(sh_scan + p_lds[j] + DP) = sk[j];
        *reinterpret_cast<float4*>(sh_scan + p_lds[j] + 2 * DP) = sa[j];
      }
#pragma unroll
    for (int j = 0; j < LA_MAX_CHUNK; ++j)
      if (j < v_slots) {
        const int i = tid + j * nthr, tt = i >> nwc_log2;
        if (tt < n) sh_scan[tt * rec + 3 * DP + (i & (NWC - 1))] = sv[j];
      }
    if (MODE == 1 && tid < n) sh_scan[tid * rec + 3 * DP + NWC] = sb;
  };
  // a token's values for this lane out of LDS
  auto read = [&](int tt, float (&q_)[R], float (&k_)[R], float (&a_)[R], float& v_,
                  float& b_) {
    const float* base = sh_scan + tt * rec;
#pragma unroll
    for (int r4 = 0; r4 < R; r4 += 4) {
      const int row = la_row<KS>(s, r4);
      const float4 x = *reinterpret_cast<const float4*>(base + row);
      const float4 y = *reinterpret_cast<const float4*>(base + DP + row);
      const float4 z = *reinterpret_cast<const float4*>(base + 2 * DP + row);
      q_[r4] = x.x; q_[r4 + 1] = x.y; q_[r4 + 2] = x.z; q_[r4 + 3] = x.w;
      k_[r4] = y.x; k_[r4 + 1] = y.y; k_[r4 + 2] = y.z; k_[r4 + 3] = y.w;
      a_[r4] = z.x; a_[r4 + 1] = z.y; a_[r4 + 2] = z.z; a_[r4 + 3] = z.w;
    }
    v_ = base[3 * DP + cl];
    b_ = base[3 * DP + NWC];
  };
  int n = min(tb, last - first);
  if (n > 0) fetch(first, n);
  // (the zeros beyond d stay; no more tokens' places than the segment will use)
  for (int i = tid; i < min(tb, last - first) * rec; i += nthr) sh_scan[i] = 0.f;
  __syncthreads();
  if (n > 0) put(n);
  __syncthreads();
  float* orow = out + (size_t)h * dv + c;
  const size_t ostep = (size_t)H * dv;
  const bool writes = s == 0 && col_ok;
  for (int t0 = first; t0 < last; t0 += tb) {
    n = min(tb, last - t0);
    const int nn = min(tb, last - t0 - tb);
    if (nn > 0) fetch(t0 + tb, nn);
    // two sets of registers take turns: one is read for the next token while the other is used
    // (a read past the chunk's tokens stays inside the chunk's LDS or the next one's start, and
    // what it brings is not used: the loop over pairs needs no tests inside)
    float q0[R], k0[R], a0[R], v0, b0, q1[R], k1[R], a1[R], v1, b1;
    float* op = orow + (size_t)t0 * ostep;
    read(0, q0, k0, a0, v0, b0);
    int tt = 0;
    for (; tt + 1 < n; tt += 2) {
      read(tt + 1, q1, k1, a1, v1, b1);
      const float o0 = la_token<KS, R, MODE>(S, q0, k0, a0, uc, v0, b0);
      if (writes) op[0] = o0;
      read(min(tt + 2, tb - 1), q0, k0, a0, v0, b0);
      const float o1 = la_token<KS, R, MODE>(S, q1, k1, a1, uc, v1, b1);
      if (writes) op[ostep] = o1;
      op += 2 * ostep;
    }
    if (tt < n) {
      const float o0 = la_token<KS, R, MODE>(S, q0, k0, a0, uc, v0, b0);
      if (writes) op[0] = o0;
    }
    __syncthreads();
    if (nn > 0) put(nn);
    __syncthreads();
  }
  if (col_ok) la_store_rows<KS, R>(st, s, d, S);
}

template <int KS, int R, int MODE, typename TV>
__global__ __launch_bounds__(WAVE) void matrix_state_scan_wave_kernel(
    const float* __restrict__ qf, const float* __restrict__ kf, const float* __restrict__ af,
    const float* __restrict__ bf, const TV* __restrict__ v, int v_stride,
    float* __restrict__ state, const int* __restrict__ seg_start,
    const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot, int H, int Hk, int d,
    int dv, float* __restrict__ out) {
  constexpr int COLS = WAVE / KS;
  const int seg = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
  const int s = lane % KS, c = blockIdx.x * COLS + lane / KS;
  const bool col_ok = c < dv;
  const int cc = col_ok ? c : dv - 1;
  const int hk = h / (H / Hk);
  const int first = seg_start[seg], last = seg_start[seg + 1];
  float* st = state + (((size_t)seg_slot[seg] * H + h) * dv + cc) * d;
  float S[R];
  la_load_rows<KS, R>(st, s, d, seg_pos0[seg] > 0, S);
  float uc[R];      // MODE 2: the lane's rows of the head's bonus, which `bf` then holds [H, d]
#pragma unroll
  for (int r = 0; r < R; ++r)
    uc[r] = MODE == 2 && la_row<KS>(s, r) < d ? bf[(size_t)h * d + la_row<KS>(s, r)] : 0.f;

  float qn[R], kn[R], an[R], vn = 0.f, bn = 0.f;
  auto fetch = [&](int t) {
    const float* qr = qf + ((size_t)t * Hk + hk) * d;
    const float* kr = kf + ((size_t)t * Hk + hk) * d;
    const float* ar = af + ((size_t)t * H + h) * d;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = la_row<KS>(s, r);
      const bool ok = row < d;
      qn[r] = ok ? qr[row] : 0.f;
      kn[r] = ok ? kr[row] : 0.f;
      an[r] = ok ? ar[row] : 0.f;
    }
    vn = to_f32(v[(size_t)t * v_stride + (size_t)h * dv + cc]);
    if (MODE == 1) bn = bf[(size_t)t * H + h];
  };
  if (first < last) fetch(first);
  for (int t = first; t < last; ++t) {
    float qc[R], kc[R], ac[R];
#pragma unroll
    for (int r = 0; r < R; ++r) { qc[r] = qn[r]; kc[r] = kn[r]; ac[r] = an[r]; }
    const float vc = vn, bc = bn;
    if (t + 1 < last) fetch(t + 1);
    const float o = la_token<KS, R, MODE>(S, qc, kc, ac, uc, vc, bc);
    if (s == 0 && col_ok) out[(size_t)t * H * dv + (size_t)h * dv + c] = o;
  }
  if (col_ok) la_store_rows<KS, R>(st, s, d, S);
}

// The block form's shape for a problem: waves a block (a power of two up to four, no more than
// the columns ask for; halved while that leaves CUs without a block), tokens a chunk (0: the
// shape does not fit and the wave form runs).
struct LaBlockShape { int nw, tb, nwc_log2, rec; };
#define LA_LDS_FLOATS 12288      // 48 KB
static LaBlockShape la_block_shape(int ks, int r, int H, int S, int T, int d, int dv) {
  const int cols = WAVE / ks, col_waves = (dv + cols - 1) / cols;
  int nw = 1;
  while (nw * 2 <= LA_MAX_WAVES && nw < col_waves) nw *= 2;
  while (nw > 2 && (long long)H * S * ((col_waves + nw - 1) / nw) < 256) nw /= 2;
  int lg = 0;
  while ((1 << lg) < nw * cols) ++lg;
  const int rec = 3 * ks * r + ((nw * cols + 1 + 3) & ~3);
  int tb = d % 4 ? 0 : LA_QS * nw * WAVE / (d / 4);
  if (tb > LA_MAX_CHUNK) tb = LA_MAX_CHUNK;
  if (tb > LA_LDS_FLOATS / rec) tb = LA_LDS_FLOATS / rec;
  if (tb > T) tb = T;                 // (no segment is longer than the step)
  return LaBlockShape{nw, tb, lg, rec};
}

template <int KS, int R, int MODE, typename TV>
static void scan_launch_typed(const float* qf, const float* kf, const float* af, const float* bf,
                              const TV* v, int v_stride, float* state, const int* seg_start,
                              const int* seg_pos0, const int* seg_slot, int T, int S, int H,
                              int Hk, int d, int dv, int form, float* out, hipStream_t stream) {
  constexpr int COLS = WAVE / KS;
  const LaBlockShape b = la_block_shape(KS, R, H, S, T, d, dv);
  if (form == 1 || b.tb < 1) {
    hipLaunchKernelGGL((matrix_state_scan_wave_kernel<KS, R, MODE, TV>),
                       dim3((dv + COLS - 1) / COLS, H, S), dim3(WAVE), 0, stream, qf, kf, af, bf,
                       v, v_stride, state, seg_start, seg_pos0, seg_slot, H, Hk, d, dv, out);
    return;
  }
  const int nwc = b.nw * COLS;
  hipLaunchKernelGGL((matrix_state_scan_block_kernel<KS, R, MODE, TV>),
                     dim3((dv + nwc - 1) / nwc, H, S), dim3(b.nw * WAVE),
                     (size_t)b.tb * b.rec * sizeof(float), stream, qf, kf, af, bf, v, v_stride,
                     state, seg_start, seg_pos0, seg_slot, H, Hk, d, dv, b.tb, b.rec, b.nwc_log2,
                     out);
}

template <int KS, int R, int MODE>
static void scan_launch(const float* qf, const float* kf, const float* af, const float* bf,
                        const void* v, int v_stride, int v_is_bf16, float* state,
                        const int* seg_start, const int* seg_pos0, const int* seg_slot, int T,
                        int S, int H, int Hk, int d, int dv, int form, float* out,
                        hipStream_t stream) {
  if (v_is_bf16)
    scan_launch_typed<KS, R, MODE, bf16_t>(qf, kf, af, bf, (const bf16_t*)v, v_stride, state,
                                         seg_start, seg_pos0, seg_slot, T, S, H, Hk, d, dv, form,
                                         out, stream);
  else
    scan_launch_typed<KS, R, MODE, float>(qf, kf, af, bf, (const float*)v, v_stride, state,
                                        seg_start, seg_pos0, seg_slot, T, S, H, Hk, d, dv, form,
                                        out, stream);
}

// form: 0 = the block form where it fits, 1 = the wave form, 2 = the block form or an error.
extern "C" int kappai_matrix_state_scan(const float* qf, const float* kf, const float* af,
                                        const float* bf, const void* v, int v_stride,
                                        int v_is_bf16, float* state, const int* seg_start,
                                        const int* seg_pos0, const int* seg_slot, int T, int S,
                                        int H, int Hk, int d, int dv, int mode, int form,
                                        float* out, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (H < 1 || Hk < 1 || H % Hk || H > 65535 || S > 65535 || d < 1 || d > 64 * 16 || dv < 1 ||
      form < 0 || form > 2 || mode < 0 || mode > 2)
    return (int)hipErrorInvalidValue;
  // mode 1 (delta rule): bf = beta [T, H]; mode 2 (bonus): bf = the bonus [H, d], H == Hk
  if (mode && bf == nullptr) return (int)hipErrorInvalidValue;
  if (mode == 2 && H != Hk) return (int)hipErrorInvalidValue;
  // eight rows a lane; sixteen for the key sizes that 64 lanes of eight do not hold
  const int r = d <= 64 * 8 ? 8 : 16;
  int ks = 1;
  while (ks * r < d) ks *= 2;
  if (form == 2 && la_block_shape(ks, r, H, S, T, d, dv).tb < 1) return (int)hipErrorInvalidValue;
#define LA_CASE(KS_, R_)                                                                          \
  case KS_ * 100 + R_:                                                                                    \
    if (mode == 1)                                                                              \
      scan_launch<KS_, R_, 1>(qf, kf, af, bf, v, v_stride, v_is_bf16, state, seg_start, seg_pos0, \
                             seg_slot, T, S, H, Hk, d, dv, form, out, stream);                     \
    else if (mode == 2)                                                                         \
      scan_launch<KS_, R_, 2>(qf, kf, af, bf, v, v_stride, v_is_bf16, state, seg_start, seg_pos0, \
                             seg_slot, T, S, H, Hk, d, dv, form, out, stream);                     \
    else                                                                                        \
      scan_launch<KS_, R_, 0>(qf, kf, af, bf, v, v_stride, v_is_bf16, state, seg_start,         \
                              seg_pos0, seg_slot, T, S, H, Hk, d, dv, form, out, stream);          \
    break;
  switch (ks * 100 + r) {
    LA_CASE(1, 8) LA_CASE(2, 8) LA_CASE(4, 8) LA_CASE(8, 8) LA_CASE(16, 8) LA_CASE(32, 8)
    LA_CASE(64, 8) LA_CASE(64, 16)
    default: return (int)hipErrorInvalidValue;
  }
#undef LA_CASE
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// One fixed decay a head, S <- lam S + k v^T, o = S^T q, over long portions in chunks of rows.
// A constant decay has a form without a chain along the tokens and without a division: inside
// a chunk of n rows  o_i = sum_(j <= i) lam^(i - j) (q_i . k_j) v_j + lam^(i + 1) S0^T q_i  with
// S0 the state the chunk starts from, and behind it  S = lam^n S0 + sum_j lam^(n - 1 - j) k_j
// v_j^T.  Every power is of a number in [0, 1] with an exponent >= 0.  Three passes, as the scans
// per channel take them: the chunks' own sums side by side; a thread an element of the state
// carries it over a segment's chunks in order, leaving in `carry` the state every chunk starts
// from; the chunks' outputs side by side.  Everything is float32 on the vector units (scores,
// their weights and the state are asked for in 32 bits): products of tiles staged in LDS so that
// the summed index is the row of both operands, a thread keeping 4 x 4 results.
// `carry` [n_chunks, H, d, dv] (a head's matrix row by row: a row of S0 is one stretch for the
// pass that multiplies by it; the state itself lies column by column).
// ---------------------------------------------------------------------------------------
#define FD_C 32         // most rows of a chunk
#define FD_T 64         // key channels / value channels a tile
#define FD_THREADS 128
#define FD_CS (FD_C + 4)   // row strides in LDS: multiples of four floats, off the powers of two
#define FD_TS (FD_T + 4)

// Element i of a tile of FD_C rows x FD_T channels that is read from rows of channels and stored
// [channel][row]: a wave's lanes take eight channels of eight rows, so that their stores fall on
// all the banks (a row stride of FD_CS floats puts neighbouring channels four banks apart).
__device__ __forceinline__ int fd_spread_e(int i) { return (i % 8) + 8 * ((i / 64) % (FD_T / 8)); }
__device__ __forceinline__ int fd_spread_j(int i) { return ((i / 8) % 8) + 8 * (i / (8 * FD_T)); }

// acc[a][b] += sum_(k < kn) X[k][a0 + a] * Y[k][b0 + b]
__device__ __forceinline__ void fd_outer(float (&acc)[4][4], const float* X, int xs, const float* Y,
                                         int ys, int a0, int b0, int kn) {
#pragma unroll 4
  for (int k = 0; k < kn; ++k) {
    const float4 x4 = *reinterpret_cast<const float4*>(X + k * xs + a0);
    const float4 y4 = *reinterpret_cast<const float4*>(Y + k * ys + b0);
    const float x[4] = {x4.x, x4.y, x4.z, x4.w}, y[4] = {y4.x, y4.y, y4.z, y4.w};
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) acc[a][b] = fmaf(x[a], y[b], acc[a][b]);
  }
}

template <typename TV>
__global__ __launch_bounds__(FD_THREADS) void fixed_decay_chunk_sums_kernel(
    const float* __restrict__ kf, const TV* __restrict__ v, int v_stride,
    const float* __restrict__ rate, const int* __restrict__ chunks, int H, int d, int dv,
    int n_ct, float* __restrict__ carry) {
  __shared__ __attribute__((aligned(16))) float Ks[FD_C][FD_T];
  __shared__ __attribute__((aligned(16))) float Vs[FD_C][FD_T];
  __shared__ float pw[FD_C + 1];
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int c0 = (blockIdx.z % n_ct) * FD_T, r0 = (blockIdx.z / n_ct) * FD_T;
  const int row0 = chunks[3 * ch + 1], n = min(chunks[3 * ch + 2], FD_C);
  if (tid <= FD_C) pw[tid] = powf(rate[h], (float)tid);
  __syncthreads();
  for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
    const int j = i / FD_T, e = i % FD_T;
    const size_t row = (size_t)(row0 + j);
    Ks[j][e] = (j < n && r0 + e < d) ? kf[(row * H + h) * d + r0 + e] * pw[n - 1 - j] : 0.f;
    Vs[j][e] = (j < n && c0 + e < dv) ? to_f32(v[row * v_stride + (size_t)h * dv + c0 + e]) : 0.f;
  }
  __syncthreads();
  for (int tile = tid; tile < (FD_T / 4) * (FD_T / 4); tile += FD_THREADS) {
    const int a0 = (tile / (FD_T / 4)) * 4, b0 = (tile % (FD_T / 4)) * 4;
    float acc[4][4] = {};
    fd_outer(acc, &Vs[0][0], FD_T, &Ks[0][0], FD_T, a0, b0, n);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int c = c0 + a0 + a, r = r0 + b0 + b;
        if (c < dv && r < d) carry[(((size_t)ch * H + h) * d + r) * dv + c] = acc[a][b];
      }
  }
}

__global__ __launch_bounds__(256) void fixed_decay_chunk_carry_kernel(
    const float* __restrict__ rate, const int* __restrict__ chunks,
    const int* __restrict__ seg_chunk0, const int* __restrict__ seg_pos0,
    const int* __restrict__ seg_slot, int H, int d, int dv, float* __restrict__ carry,
    float* __restrict__ state) {
  const int seg = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x, n_el = dv * d;
  if (e >= n_el) return;
  const int ch0 = seg_chunk0[seg], ch1 = seg_chunk0[seg + 1];
  if (ch0 >= ch1) return;
  const float lam = rate[h], lam_full = powf(lam, (float)FD_C);
  float* st = state + ((size_t)seg_slot[seg] * H + h) * n_el + (size_t)(e % dv) * d + e / dv;
  float S = seg_pos0[seg] > 0 ? *st : 0.f;
  for (int c = ch0; c < ch1; c += 4) {
    float own[4];
    int rows[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int cc = min(c + i, ch1 - 1);
      own[i] = carry[((size_t)cc * H + h) * n_el + e];
      rows[i] = chunks[3 * cc + 2];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (c + i >= ch1) break;
      carry[((size_t)(c + i) * H + h) * n_el + e] = S;      // the state the chunk starts from
      S = fmaf(rows[i] == FD_C ? lam_full : powf(lam, (float)rows[i]), S, own[i]);
    }
  }
  *st = S;
}

template <typename TV>
__global__ __launch_bounds__(FD_THREADS) void fixed_decay_chunk_out_kernel(
    const float* __restrict__ qf, const float* __restrict__ kf, const TV* __restrict__ v,
    int v_stride, const float* __restrict__ rate, const int* __restrict__ chunks, int H, int d,
    int dv, const float* __restrict__ carry, float* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) float Qt[FD_T][FD_CS];     // [key channel][row]
  __shared__ __attribute__((aligned(16))) float Kt[FD_T][FD_CS];
  __shared__ __attribute__((aligned(16))) float Pt[FD_C][FD_CS];     // [key row j][query row i]
  __shared__ __attribute__((aligned(16))) float Vs[FD_C][FD_T];      // [row][value channel]
  __shared__ __attribute__((aligned(16))) float St[FD_T][FD_TS];     // [key channel][value channel]
  __shared__ float pw[FD_C + 1];
  const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * FD_T, tid = threadIdx.x;
  const int row0 = chunks[3 * ch + 1], n = min(chunks[3 * ch + 2], FD_C);
  if (tid <= FD_C) pw[tid] = powf(rate[h], (float)tid);
  // the scores of the chunk, P[i][j] = q_i . k_j: 64 tiles of 4 x 4, one wave
  const int pi0 = (tid / (FD_C / 4)) * 4, pj0 = (tid % (FD_C / 4)) * 4;
  float accP[4][4] = {};
  for (int r0 = 0; r0 < d; r0 += FD_T) {
    __syncthreads();
    for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
      const int e = fd_spread_e(i), j = fd_spread_j(i);
      const bool ok = j < n && r0 + e < d;
      const size_t at = ((size_t)(row0 + j) * H + h) * d + r0 + e;
      Qt[e][j] = ok ? qf[at] : 0.f;
      Kt[e][j] = ok ? kf[at] : 0.f;
    }
    __syncthreads();
    if (tid < (FD_C / 4) * (FD_C / 4))
      fd_outer(accP, &Qt[0][0], FD_CS, &Kt[0][0], FD_CS, pi0, pj0, min(FD_T, d - r0));
  }
  if (tid < (FD_C / 4) * (FD_C / 4)) {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int i = pi0 + a, j = pj0 + b;
        Pt[j][i] = (j <= i && i < n) ? accP[a][b] * pw[i - j] : 0.f;
      }
  }
  for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
    const int j = i / FD_T, e = i % FD_T;
    Vs[j][e] = (j < n && c0 + e < dv)
                   ? to_f32(v[(size_t)(row0 + j) * v_stride + (size_t)h * dv + c0 + e]) : 0.f;
  }
  __syncthreads();
  // the outputs, 32 rows x 64 value channels: 128 tiles of 4 x 4
  const int oi0 = (tid / (FD_T / 4)) * 4, oc0 = (tid % (FD_T / 4)) * 4;
  float accO[4][4] = {}, accS[4][4] = {};
  fd_outer(accO, &Pt[0][0], FD_CS, &Vs[0][0], FD_T, oi0, oc0, n);
  const float* S0 = carry + ((size_t)ch * H + h) * dv * d;
  for (int r0 = 0; r0 < d; r0 += FD_T) {
    __syncthreads();
    for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
      const int e = fd_spread_e(i), j = fd_spread_j(i);
      Qt[e][j] = (j < n && r0 + e < d) ? qf[((size_t)(row0 + j) * H + h) * d + r0 + e] : 0.f;
    }
    if (dv % 4 == 0) {
      for (int i = tid; i < FD_T * FD_T / 4; i += FD_THREADS) {
        const int e = i / (FD_T / 4), c = (i % (FD_T / 4)) * 4;
        float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c0 + c < dv && r0 + e < d)
          s4 = *reinterpret_cast<const float4*>(S0 + (size_t)(r0 + e) * dv + c0 + c);
        *reinterpret_cast<float4*>(&St[e][c]) = s4;
      }
    } else {
      for (int i = tid; i < FD_T * FD_T; i += FD_THREADS) {
        const int e = i / FD_T, c = i % FD_T;
        St[e][c] = (c0 + c < dv && r0 + e < d) ? S0[(size_t)(r0 + e) * dv + c0 + c] : 0.f;
      }
    }
    __syncthreads();
    fd_outer(accS, &Qt[0][0], FD_CS, &St[0][0], FD_TS, oi0, oc0, min(FD_T, d - r0));
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int i = oi0 + a;
    if (i >= n) continue;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int c = c0 + oc0 + b;
      if (c < dv)
        out[((size_t)(row0 + i) * H + h) * dv + c] = fmaf(pw[i + 1], accS[a][b], accO[a][b]);
    }
  }
}

// qf, kf [T, H, d] float32 as recurrence_prep leaves them, v [T, >= H dv] with a row stride,
// rate [H] the decays, chunks [n_chunks, 3] = (segment, first row, rows <= 32), seg_chunk0
// [S + 1], carry [n_chunks, H, d, dv] floats of scratch, state [slots, H, dv, d], out [T, H dv].
extern "C" int kappai_fixed_decay_chunks(const float* qf, const float* kf, const void* v,
                                         int v_stride, int v_is_bf16, const float* rate,
                                         float* state, const int* seg_pos0, const int* seg_slot,
                                         const int* chunks, const int* seg_chunk0, int n_chunks,
                                         int chunk_rows, int T, int S, int H, int d, int dv,
                                         float* carry, float* out, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (H < 1 || H > 65535 || d < 1 || dv < 1 || n_chunks < 1 ||
      chunk_rows < 1 || chunk_rows > FD_C || !chunks || !seg_chunk0 || !carry || !rate)
    return (int)hipErrorInvalidValue;
  const int n_ct = (dv + FD_T - 1) / FD_T, n_rt = (d + FD_T - 1) / FD_T;
  const int el_blocks = (dv * d + 255) / 256;
  if (n_ct * n_rt > 65535 || el_blocks > 65535) return (int)hipErrorInvalidValue;
  const dim3 sums(n_chunks, H, n_ct * n_rt), outs(n_chunks, H, n_ct);
  if (v_is_bf16)
    hipLaunchKernelGGL(fixed_decay_chunk_sums_kernel<bf16_t>, sums, dim3(FD_THREADS), 0, stream,
                       kf, (const bf16_t*)v, v_stride, rate, chunks, H, d, dv, n_ct, carry);
  else
    hipLaunchKernelGGL(fixed_decay_chunk_sums_kernel<float>, sums, dim3(FD_THREADS), 0, stream,
                       kf, (const float*)v, v_stride, rate, chunks, H, d, dv, n_ct, carry);
  hipLaunchKernelGGL(fixed_decay_chunk_carry_kernel, dim3(S, H, el_blocks), dim3(256), 0, stream,
                     rate, chunks, seg_chunk0, seg_pos0, seg_slot, H, d, dv, carry, state);
  if (v_is_bf16)
    hipLaunchKernelGGL(fixed_decay_chunk_out_kernel<bf16_t>, outs, dim3(FD_THREADS), 0, stream,
                       qf, kf, (const bf16_t*)v, v_stride, rate, chunks, H, d, dv, carry, out);
  else
    hipLaunchKernelGGL(fixed_decay_chunk_out_kernel<float>, outs, dim3(FD_THREADS), 0, stream,
                       qf, kf, (const float*)v, v_stride, rate, chunks, H, d, dv, carry, out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// A decay per token and key channel with the bonus for the own token, over long portions in
// chunks of rows: o_i = (S_(i-1) + diag(u) k_i v_i^T)^T q_i, S_i = diag(a_i) S_(i-1) + k_i v_i^T.
// With L_j = log a_0 + .. + log a_j inside the chunk (L_(-1) = 0) and S0 the state the chunk
// starts from,
//   o_i = sum_(j < i) [sum_r q_i[r] k_j[r] exp(L_(i-1)[r] - L_j[r])] v_j + (q_i . (u * k_i)) v_i
//         + S0^T (q_i * exp(L_(i-1)))
//   S   = diag(exp(L_(n-1))) S0 + sum_j (k_j * exp(L_(n-1) - L_j)) v_j^T.
// Every exponent is a sum of logarithms of decays, so <= 0: nothing is ever divided by a decay.
// The weights inside the brackets are made term by term on the vector units (an exponential a
// term); everything else is the products of tiles of the fixed decay's kernels, and the same
// three passes.  A decay that has underflowed to zero counts as exp(-200), which is zero again in
// float32 while its logarithm stays finite.  `total` [n_chunks, H, d]: exp(L_(n-1)) of a chunk.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float fd_log_decay(float a) { return fmaxf(logf(a), -104.f); }

template <typename TV>
__global__ __launch_bounds__(FD_THREADS) void channel_decay_chunk_sums_kernel(
    const float* __restrict__ kf, const float* __restrict__ af, const TV* __restrict__ v,
    int v_stride, const int* __restrict__ chunks, int H, int d, int dv, int n_ct,
    float* __restrict__ carry, float* __restrict__ total) {
  __shared__ __attribute__((aligned(16))) float Ks[FD_C][FD_T];
  __shared__ __attribute__((aligned(16))) float Vs[FD_C][FD_T];
  __shared__ float Ls[FD_C][FD_T];
  __shared__ float Ln[FD_T];
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int ct = blockIdx.z % n_ct, c0 = ct * FD_T, r0 = (blockIdx.z / n_ct) * FD_T;
  const int row0 = chunks[3 * ch + 1], n = min(chunks[3 * ch + 2], FD_C);
  if (tid < FD_T) {
    float run = 0.f;
    const bool ok = r0 + tid < d;
    for (int j = 0; j < n; ++j) {
      if (ok) run += fd_log_decay(af[((size_t)(row0 + j) * H + h) * d + r0 + tid]);
      Ls[j][tid] = run;
    }
    Ln[tid] = run;
    if (ct == 0 && ok) total[((size_t)ch * H + h) * d + r0 + tid] = expf(run);
  }
  __syncthreads();
  for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
    const int j = i / FD_T, e = i % FD_T;
    const size_t row = (size_t)(row0 + j);
    Ks[j][e] = (j < n && r0 + e < d)
                   ? kf[(row * H + h) * d + r0 + e] * expf(fminf(Ln[e] - Ls[j][e], 0.f)) : 0.f;
    Vs[j][e] = (j < n && c0 + e < dv) ? to_f32(v[row * v_stride + (size_t)h * dv + c0 + e]) : 0.f;
  }
  __syncthreads();
  for (int tile = tid; tile < (FD_T / 4) * (FD_T / 4); tile += FD_THREADS) {
    const int a0 = (tile / (FD_T / 4)) * 4, b0 = (tile % (FD_T / 4)) * 4;
    float acc[4][4] = {};
    fd_outer(acc, &Vs[0][0], FD_T, &Ks[0][0], FD_T, a0, b0, n);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int c = c0 + a0 + a, r = r0 + b0 + b;
        if (c < dv && r < d) carry[(((size_t)ch * H + h) * d + r) * dv + c] = acc[a][b];
      }
  }
}

__global__ __launch_bounds__(256) void channel_decay_chunk_carry_kernel(
    const float* __restrict__ total, const int* __restrict__ seg_chunk0,
    const int* __restrict__ seg_pos0, const int* __restrict__ seg_slot, int H, int d, int dv,
    float* __restrict__ carry, float* __restrict__ state) {
  const int seg = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x, n_el = dv * d;
  if (e >= n_el) return;
  const int ch0 = seg_chunk0[seg], ch1 = seg_chunk0[seg + 1];
  if (ch0 >= ch1) return;
  const int r = e / dv;
  float* st = state + ((size_t)seg_slot[seg] * H + h) * n_el + (size_t)(e % dv) * d + r;
  float S = seg_pos0[seg] > 0 ? *st : 0.f;
  for (int c = ch0; c < ch1; c += 4) {
    float own[4], fac[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int cc = min(c + i, ch1 - 1);
      own[i] = carry[((size_t)cc * H + h) * n_el + e];
      fac[i] = total[((size_t)cc * H + h) * d + r];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (c + i >= ch1) break;
      carry[((size_t)(c + i) * H + h) * n_el + e] = S;      // the state the chunk starts from
      S = fmaf(fac[i], S, own[i]);
    }
  }
  *st = S;
}

template <typename TV>
__global__ __launch_bounds__(FD_THREADS) void channel_decay_chunk_out_kernel(
    const float* __restrict__ qf, const float* __restrict__ kf, const float* __restrict__ af,
    const TV* __restrict__ v, int v_stride, const float* __restrict__ bonus,
    const int* __restrict__ chunks, int H, int d, int dv, const float* __restrict__ carry,
    float* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) float Qt[FD_T][FD_CS];     // [key channel][row]
  __shared__ __attribute__((aligned(16))) float Kt[FD_T][FD_CS];
  // Lx[r][0] = 0, Lx[r][j + 1] = L_j: row i reads L_(i-1) at [i], key row j its L_j at [j + 1]
  __shared__ __attribute__((aligned(16))) float Lx[FD_T][FD_CS];
  __shared__ __attribute__((aligned(16))) float Pt[FD_C][FD_CS];     // [key row j][query row i]
  __shared__ __attribute__((aligned(16))) float Vs[FD_C][FD_T];      // [row][value channel]
  __shared__ __attribute__((aligned(16))) float St[FD_T][FD_TS];     // [key channel][value channel]
  const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * FD_T, tid = threadIdx.x;
  const int row0 = chunks[3 * ch + 1], n = min(chunks[3 * ch + 2], FD_C);
  // the weights of the chunk's own rows: 128 tiles of 4 rows i x 2 rows j
  const int pi0 = (tid / (FD_C / 2)) * 4, pj0 = (tid % (FD_C / 2)) * 2;
  const bool p_live = pj0 < pi0 + 3;            // (a tile with some j < i)
  float accP[4][2] = {}, diag = 0.f;
  // the outputs, 32 rows x 64 value channels: 128 tiles of 4 x 4
  const int oi0 = (tid / (FD_T / 4)) * 4, oc0 = (tid % (FD_T / 4)) * 4;
  float accO[4][4] = {}, accS[4][4] = {};
  const float* S0 = carry + ((size_t)ch * H + h) * dv * d;
  for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
    const int j = i / FD_T, e = i % FD_T;
    Vs[j][e] = (j < n && c0 + e < dv)
                   ? to_f32(v[(size_t)(row0 + j) * v_stride + (size_t)h * dv + c0 + e]) : 0.f;
  }
  for (int r0 = 0; r0 < d; r0 += FD_T) {
    const int kn = min(FD_T, d - r0);
    __syncthreads();
    for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
      const int e = fd_spread_e(i), j = fd_spread_j(i);
      const bool ok = j < n && r0 + e < d;
      const size_t at = ((size_t)(row0 + j) * H + h) * d + r0 + e;
      Qt[e][j] = ok ? qf[at] : 0.f;
      Kt[e][j] = ok ? kf[at] : 0.f;
    }
    if (tid < FD_T) {
      float run = 0.f;
      Lx[tid][0] = 0.f;
      const bool ok = r0 + tid < d;
      for (int j = 0; j < FD_C; ++j) {
        if (ok && j < n) run += fd_log_decay(af[((size_t)(row0 + j) * H + h) * d + r0 + tid]);
        Lx[tid][j + 1] = run;
      }
    }
    __syncthreads();
    if (p_live) {
#pragma unroll 2
      for (int r = 0; r < kn; ++r) {
        const float4 q4 = *reinterpret_cast<const float4*>(&Qt[r][pi0]);
        const float4 e4 = *reinterpret_cast<const float4*>(&Lx[r][pi0]);
        const float q[4] = {q4.x, q4.y, q4.z, q4.w}, e[4] = {e4.x, e4.y, e4.z, e4.w};
        const float k[2] = {Kt[r][pj0], Kt[r][pj0 + 1]};
        const float l[2] = {Lx[r][pj0 + 1], Lx[r][pj0 + 2]};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b)
            accP[a][b] = fmaf(q[a] * k[b], __expf(fminf(e[a] - l[b], 0.f)), accP[a][b]);
      }
    }
    if (tid < FD_C) {
      const float* u = bonus + (size_t)h * d + r0;
      for (int r = 0; r < kn; ++r) diag = fmaf(Qt[r][tid] * Kt[r][tid], u[r], diag);
    }
    __syncthreads();
    for (int i = tid; i < FD_C * FD_T; i += FD_THREADS) {
      const int e = i / FD_C, j = i % FD_C;
      Qt[e][j] *= expf(Lx[e][j]);
    }
    if (dv % 4 == 0) {
      for (int i = tid; i < FD_T * FD_T / 4; i += FD_THREADS) {
        const int e = i / (FD_T / 4), c = (i % (FD_T / 4)) * 4;
        float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c0 + c < dv && r0 + e < d)
          s4 = *reinterpret_cast<const float4*>(S0 + (size_t)(r0 + e) * dv + c0 + c);
        *reinterpret_cast<float4*>(&St[e][c]) = s4;
      }
    } else {
      for (int i = tid; i < FD_T * FD_T; i += FD_THREADS) {
        const int e = i / FD_T, c = i % FD_T;
        St[e][c] = (c0 + c < dv && r0 + e < d) ? S0[(size_t)(r0 + e) * dv + c0 + c] : 0.f;
      }
    }
    __syncthreads();
    fd_outer(accS, &Qt[0][0], FD_CS, &St[0][0], FD_TS, oi0, oc0, kn);
  }
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int i = pi0 + a, j = pj0 + b;
      Pt[j][i] = (j < i && i < n) ? accP[a][b] : 0.f;
    }
  __syncthreads();
  if (tid < FD_C) Pt[tid][tid] = tid < n ? diag : 0.f;
  __syncthreads();
  fd_outer(accO, &Pt[0][0], FD_CS, &Vs[0][0], FD_T, oi0, oc0, n);
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int i = oi0 + a;
    if (i >= n) continue;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int c = c0 + oc0 + b;
      if (c < dv) out[((size_t)(row0 + i) * H + h) * dv + c] = accO[a][b] + accS[a][b];
    }
  }
}

// As kappai_fixed_decay_chunks, with af [T, H, d] the decays as recurrence_prep leaves them,
// bonus [H, d], and total [n_chunks, H, d] floats of scratch beside carry.
extern "C" int kappai_channel_decay_chunks(const float* qf, const float* kf, const float* af,
                                           const void* v, int v_stride, int v_is_bf16,
                                           const float* bonus, float* state, const int* seg_pos0,
                                           const int* seg_slot, const int* chunks,
                                           const int* seg_chunk0, int n_chunks, int chunk_rows,
                                           int T, int S, int H, int d, int dv, float* carry,
                                           float* total, float* out, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (H < 1 || H > 65535 || d < 1 || dv < 1 || n_chunks < 1 || chunk_rows < 1 ||
      chunk_rows > FD_C || !chunks || !seg_chunk0 || !carry || !total || !bonus || !af)
    return (int)hipErrorInvalidValue;
  const int n_ct = (dv + FD_T - 1) / FD_T, n_rt = (d + FD_T - 1) / FD_T;
  const int el_blocks = (dv * d + 255) / 256;
  if (n_ct * n_rt > 65535 || el_blocks > 65535) return (int)hipErrorInvalidValue;
  const dim3 sums(n_chunks, H, n_ct * n_rt), outs(n_chunks, H, n_ct);
  if (v_is_bf16)
    hipLaunchKernelGGL(channel_decay_chunk_sums_kernel<bf16_t>, sums, dim3(FD_THREADS), 0, stream,
                       kf, af, (const bf16_t*)v, v_stride, chunks, H, d, dv, n_ct, carry, total);
  else
    hipLaunchKernelGGL(channel_decay_chunk_sums_kernel<float>, sums, dim3(FD_THREADS), 0, stream,
                       kf, af, (const float*)v, v_stride, chunks, H, d, dv, n_ct, carry, total);
  hipLaunchKernelGGL(channel_decay_chunk_carry_kernel, dim3(S, H, el_blocks), dim3(256), 0,
                     stream, total, seg_chunk0, seg_pos0, seg_slot, H, d, dv, carry, state);
  if (v_is_bf16)
    hipLaunchKernelGGL(channel_decay_chunk_out_kernel<bf16_t>, outs, dim3(FD_THREADS), 0, stream,
                       qf, kf, af, (const bf16_t*)v, v_stride, bonus, chunks, H, d, dv, carry,
                       out);
  else
    hipLaunchKernelGGL(channel_decay_chunk_out_kernel<float>, outs, dim3(FD_THREADS), 0, stream,
                       qf, kf, af, (const float*)v, v_stride, bonus, chunks, H, d, dv, carry,
                       out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// Per head: o / sqrt(mean(o^2) + eps) * weight[dv] * gate, gate = silu(g) (kind 0) or sigmoid(g)
// (kind 1) of the projection g [T, >= H dv] with a row stride.  A wave a (row, head).
// weight_stride: 0 when the heads share one weight [dv], dv when each has its own [H, dv].
// ---------------------------------------------------------------------------------------
#define HNG_WIDE_THREADS 256      // heads of more than 512 values take a block of four waves
template <typename T>
__global__ __launch_bounds__(HNG_WIDE_THREADS) void head_norm_gate_kernel(
    const float* __restrict__ o, const float* __restrict__ weight, float eps,
    const T* __restrict__ g, int g_stride, int gate_kind, int H, int dv, int weight_stride,
    T* __restrict__ out) {
  __shared__ float part[HNG_WIDE_THREADS / WAVE];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int threads = blockDim.x;
  weight += (size_t)h * weight_stride;
  const float* orow = o + ((size_t)t * H + h) * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += threads) ss = fmaf(orow[e], orow[e], ss);
  ss = wave_sum(ss);
  if (threads > WAVE) {
    if (lane % WAVE == 0) part[lane / WAVE] = ss;
    __syncthreads();
    ss = 0.f;
    for (int w = 0; w < threads / WAVE; ++w) ss += part[w];
  }
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  const T* gr = g + (size_t)t * g_stride + (size_t)h * dv;
  for (int e = lane; e < dv; e += threads) {
    const float gv = to_f32(gr[e]);
    const float gate = gate_kind == 0 ? gv * la_sigmoid(gv) : la_sigmoid(gv);
    from_f32(out + ((size_t)t * H + h) * dv + e, orow[e] * inv * weight[e] * gate);
  }
}

extern "C" int kappai_head_norm_gate(const float* o, const float* weight, float eps, const void* g,
                                     int g_stride, int gate_kind, int T, int H, int dv,
                                     int weight_stride, void* out, int is_bf16,
                                     hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || H > 65535 || dv < 1 || gate_kind < 0 || gate_kind > 1)
    return (int)hipErrorInvalidValue;
  const dim3 block(dv > 512 ? HNG_WIDE_THREADS : WAVE);
  if (is_bf16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, dim3(T, H), block, 0, stream, o, weight,
                       eps, (const bf16_t*)g, g_stride, gate_kind, H, dv, weight_stride, (bf16_t*)out);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3(T, H), block, 0, stream, o, weight,
                       eps, (const float*)g, g_stride, gate_kind, H, dv, weight_stride, (float*)out);
  KAPPAI_RETURN_LAUNCH_STATUS();
}
