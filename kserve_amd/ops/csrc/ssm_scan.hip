// State-space (Mamba-2 / SSD form) sequence mixer kernels over a flat,
// variable-length token batch with per-sequence state slots.
//
// A sequence's portion may start anywhere: `positions[t]` is the absolute
// position of token t, `seq_of_token[t]` its sequence in the batch,
// `cu_seqlens[s]` the first flat token of sequence s and `slots[s]` the row
// of the state pools that carries it between steps. A portion that starts at
// position 0 ignores whatever its slot held (slots are reused, never cleared).
//
//  * causal_conv_silu: depthwise causal convolution over `taps` inputs per
//    channel + bias + silu. Inputs before the portion come from the conv
//    state (the last taps-1 raw inputs of the sequence), zeros before
//    position 0.
//  * conv_state_update: runs after the above, shifts the new raw inputs in.
//  * ssd_scan: per head h with group g(h):
//        a_t = exp(-exp(A_log_h) * dt_t),  dt_t = softplus(dt_raw + dt_bias_h)
//        S_t = a_t S_{t-1} + dt_t B_t x_t^T        (S: N x P, fp32)
//        y_t = S_t^T C_t + D_h x_t
//    The state lives in registers: lane (ns, p) owns rows n = ns + 16 r of
//    column p, a 16-lane shuffle tree sums the C-contraction. Tokens of a
//    sequence are walked in order with the next token's operands in flight.
//    Serves prefill portions and single-token decode alike (grid = sequences
//    x heads x column tiles, so decode batches fill the chip).
#include "dtype_io.h"

namespace {

constexpr int MAX_TAPS = 16;

__device__ __forceinline__ float silu_f(float v) {
  return v / (1.0f + expf(-v));
}

template <typename T>
__global__ void causal_conv_silu_kernel(
    float* __restrict__ out, const T* __restrict__ in, long in_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ conv_state, const long* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int channels, int taps) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int s = seq_of_token[t];
  const int first = cu_seqlens[s];
  const long pos = positions[t];
  const long slot = slots[s];
  const int hist = taps - 1;
  float acc = bias[c];
  for (int j = 0; j < taps; ++j) {
    const int back = hist - j;  // 0 = the current token
    if (pos - back < 0) continue;
    float v;
    if (t - back >= first) {
      v = ld_f32(in, (long)(t - back) * in_stride + c);
    } else {
      // state row i holds the input at position (portion start - hist + i)
      const int i = hist - back + (t - first);
      v = ld_f32(conv_state, (slot * hist + i) * channels + c);
    }
    acc += w[(long)c * taps + j] * v;
  }
  out[(long)t * channels + c] = silu_f(acc);
}

template <typename T>
__global__ void conv_state_update_kernel(
    T* __restrict__ conv_state, const T* __restrict__ in, long in_stride,
    const long* __restrict__ positions, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int channels, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = cu_seqlens[s];
  const int len = cu_seqlens[s + 1] - first;
  if (len <= 0) return;
  const long start = positions[first];
  const long slot = slots[s];
  const int hist = taps - 1;
  T keep[MAX_TAPS];
  // new row i holds position (start + len - hist + i)
  for (int i = 0; i < hist; ++i) {
    const long rel = (long)len - hist + i;  // offset into the portion
    T v;
    if (rel >= 0) {
      v = in[(first + rel) * in_stride + c];
    } else if (start + rel < 0) {
      st_f32(&v, 0, 0.f);
    } else {
      v = conv_state[(slot * hist + (hist + rel)) * channels + c];
    }
    keep[i] = v;
  }
  for (int i = 0; i < hist; ++i)
    conv_state[(slot * hist + i) * channels + c] = keep[i];
}

// R = state rows per lane (N <= 16 R); blockDim = 256 = 16 ns-lanes x 16 cols
template <int R>
__global__ void __launch_bounds__(256) ssd_scan_kernel(
    float* __restrict__ y, const float* __restrict__ xbc,
    const float* __restrict__ dt_raw_f32, const short* __restrict__ dt_raw_bf16,
    long dt_stride, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip,
    float* __restrict__ state, const long* __restrict__ positions,
    const int* __restrict__ cu_seqlens, const int* __restrict__ slots,
    int heads, int groups, int P, int N) {
  const int s = blockIdx.z;
  const int h = blockIdx.y;
  const int ns = threadIdx.x & 15;
  const int p = blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool p_ok = p < P;
  const int first = cu_seqlens[s];
  const int len = cu_seqlens[s + 1] - first;
  if (len <= 0) return;
  const int g = h / (heads / groups);
  const int inner = heads * P;
  const int channels = inner + 2 * groups * N;
  const long slot = slots[s];
  const bool fresh = positions[first] == 0;
  const float A = -expf(a_log[h]);
  const float bias = dt_bias[h];
  const float Dh = d_skip[h];

  float S[R];
  float* sp = state + ((slot * heads + h) * (long)P + (p_ok ? p : 0)) * N;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = ns + 16 * r;
    S[r] = (!fresh && p_ok && n < N) ? sp[n] : 0.f;
  }

  auto load_dt = [&](int t) -> float {
    const long i = (long)t * dt_stride + h;
    return dt_raw_f32 ? dt_raw_f32[i] : bf16_bits_to_float(dt_raw_bf16[i]);
  };

  // operands of the token being processed, and of the next one (prefetch)
  float Bn[R], Cn[R], xn, dtn;
  auto fetch = [&](int t) {
    const float* row = xbc + (long)t * channels;
    xn = p_ok ? row[h * P + p] : 0.f;
    dtn = load_dt(t);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = ns + 16 * r;
      const bool ok = n < N;
      Bn[r] = ok ? row[inner + g * N + n] : 0.f;
      Cn[r] = ok ? row[inner + groups * N + g * N + n] : 0.f;
    }
  };
  fetch(first);
  for (int i = 0; i < len; ++i) {
    const int t = first + i;
    float B[R], C[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      B[r] = Bn[r];
      C[r] = Cn[r];
    }
    const float x = xn;
    const float v = dtn + bias;
    if (i + 1 < len) fetch(t + 1);
    // softplus without a clamp; log1p(exp(v)) overflows only past v ~ 88
    const float dt = v > 30.f ? v : log1pf(expf(v));
    const float a = expf(A * dt);
    const float dtx = dt * x;
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] = a * S[r] + B[r] * dtx;
      acc += S[r] * C[r];
    }
    acc = group_reduce_sum<16>(acc);
    if (ns == 0 && p_ok) y[(long)t * inner + h * P + p] = acc + Dh * x;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = ns + 16 * r;
    if (p_ok && n < N) sp[n] = S[r];
  }
}

}  // namespace

extern "C" hipError_t ks_causal_conv_silu(
    void* out, const void* in, long in_stride, const void* w, const void* bias,
    void* conv_state, const void* positions, const void* seq_of_token,
    const void* cu_seqlens, const void* slots, int tokens, int num_seqs,
    int channels, int taps, int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (taps < 1 || taps > MAX_TAPS) return hipErrorInvalidValue;
  dim3 grid(cdiv(channels, 256), tokens);
  dim3 grid_u(cdiv(channels, 256), num_seqs);
  if (is_f32) {
    hipLaunchKernelGGL(causal_conv_silu_kernel<float>, grid, dim3(256), 0,
                       stream, (float*)out, (const float*)in, in_stride,
                       (const float*)w, (const float*)bias,
                       (const float*)conv_state, (const long*)positions,
                       (const int*)seq_of_token, (const int*)cu_seqlens,
                       (const int*)slots, channels, taps);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<float>, grid_u, dim3(256), 0,
                         stream, (float*)conv_state, (const float*)in,
                         in_stride, (const long*)positions,
                         (const int*)cu_seqlens, (const int*)slots, channels,
                         taps);
  } else {
    hipLaunchKernelGGL(causal_conv_silu_kernel<short>, grid, dim3(256), 0,
                       stream, (float*)out, (const short*)in, in_stride,
                       (const float*)w, (const float*)bias,
                       (const short*)conv_state, (const long*)positions,
                       (const int*)seq_of_token, (const int*)cu_seqlens,
                       (const int*)slots, channels, taps);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<short>, grid_u, dim3(256), 0,
                         stream, (short*)conv_state, (const short*)in,
                         in_stride, (const long*)positions,
                         (const int*)cu_seqlens, (const int*)slots, channels,
                         taps);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

#define SSD_LAUNCH(RR)                                                        \
  hipLaunchKernelGGL(ssd_scan_kernel<RR>, grid, dim3(256), 0, stream,         \
                     (float*)y, (const float*)xbc,                            \
                     dt_is_f32 ? (const float*)dt_raw : nullptr,              \
                     dt_is_f32 ? nullptr : (const short*)dt_raw, dt_stride,   \
                     (const float*)dt_bias, (const float*)a_log,              \
                     (const float*)d_skip, (float*)state,                     \
                     (const long*)positions, (const int*)cu_seqlens,          \
                     (const int*)slots, heads, groups, P, N)

extern "C" hipError_t ks_ssd_scan(void* y, const void* xbc, const void* dt_raw,
                                  long dt_stride, int dt_is_f32,
                                  const void* dt_bias, const void* a_log,
                                  const void* d_skip, void* state,
                                  const void* positions,
                                  const void* cu_seqlens, const void* slots,
                                  int num_seqs, int heads, int groups, int P,
                                  int N, hipStream_t stream) {
  if (num_seqs == 0) return hipSuccess;
  if (groups <= 0 || heads % groups != 0 || N < 1 || N > 256)
    return hipErrorInvalidValue;
  dim3 grid(cdiv(P, 16), heads, num_seqs);
  const int R = cdiv(N, 16);
  if (R <= 1) SSD_LAUNCH(1);
  else if (R <= 2) SSD_LAUNCH(2);
  else if (R <= 3) SSD_LAUNCH(3);
  else if (R <= 4) SSD_LAUNCH(4);
  else if (R <= 6) SSD_LAUNCH(6);
  else if (R <= 8) SSD_LAUNCH(8);
  else SSD_LAUNCH(16);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
