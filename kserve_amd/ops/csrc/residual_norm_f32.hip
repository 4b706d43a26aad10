// Norms over an fp32 residual stream, plus the embedding that starts it.
//
//  * embed_scale_sinpos: row = table[token] * scale + interleaved sinusoid
//    (even entry sin, odd entry cos of position * inv_freq[i]); fp32 out.
//  * add_rms_norm_f32res: residual += s0*d0 + s1*d1 (fp32, in place), then
//    out = residual / sqrt(mean(residual^2) + eps) * (w_offset + w).
//    The deltas are sublayer outputs in the activation dtype; either may be
//    absent. One kernel covers "add the previous sublayer, norm for the next".
//  * gated_group_rms_norm: v = y * silu(z), normalised separately in equal
//    contiguous groups of the row, times a weight (gate before the norm).
//
// Everything is accumulated in fp32 with exact (non-approximate) sqrt and
// division: these ops sit on the 32-bit path of the models that use them.
#include "dtype_io.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;

template <typename T>
__global__ void embed_scale_sinpos_kernel(float* __restrict__ out,
                                          const T* __restrict__ table,
                                          const long* __restrict__ tokens,
                                          const long* __restrict__ positions,
                                          const float* __restrict__ inv_freq,
                                          float scale, int width) {
  const long t = blockIdx.x;
  const long tok = tokens[t];
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < width; i += NT) {
    const float ang = pos * inv_freq[i >> 1];
    const float pe = (i & 1) ? cosf(ang) : sinf(ang);
    out[t * width + i] = ld_f32(table, tok * width + i) * scale + pe;
  }
}

template <typename TD, typename TO>
__global__ void add_rms_norm_f32res_kernel(
    float* __restrict__ residual, const TD* __restrict__ d0, long d0_stride,
    float s0, const TD* __restrict__ d1, long d1_stride, float s1,
    const float* __restrict__ weight, float w_offset, float eps,
    TO* __restrict__ out, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    float v = r[i];
    if (d0) v += s0 * ld_f32(d0, row * d0_stride + i);
    if (d1) v += s1 * ld_f32(d1, row * d1_stride + i);
    if (d0 || d1) r[i] = v;
    ss += v * v;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  if (!out) return;
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += NT) {
    // each thread re-reads only what it wrote itself
    st_f32(out, row * width + i, r[i] * inv * (w_offset + weight[i]));
  }
}

template <typename TZ, typename TO>
__global__ void gated_group_rms_norm_kernel(TO* __restrict__ out,
                                            const float* __restrict__ y,
                                            const TZ* __restrict__ z,
                                            long z_stride,
                                            const float* __restrict__ weight,
                                            float eps, int inner,
                                            int group_size) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  const int g0 = blockIdx.y * group_size;
  float ss = 0.f;
  for (int i = threadIdx.x; i < group_size; i += NT) {
    const float zf = ld_f32(z, row * z_stride + g0 + i);
    const float v = y[row * inner + g0 + i] * (zf / (1.0f + expf(-zf)));
    ss += v * v;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)group_size + eps);
  for (int i = threadIdx.x; i < group_size; i += NT) {
    const float zf = ld_f32(z, row * z_stride + g0 + i);
    const float v = y[row * inner + g0 + i] * (zf / (1.0f + expf(-zf)));
    st_f32(out, row * inner + g0 + i, v * inv * weight[g0 + i]);
  }
}

}  // namespace

extern "C" hipError_t ks_embed_scale_sinpos(void* out, const void* table,
                                            const void* tokens,
                                            const void* positions,
                                            const void* inv_freq, float scale,
                                            int rows, int width, int is_f32,
                                            hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (is_f32)
    hipLaunchKernelGGL(embed_scale_sinpos_kernel<float>, dim3(rows), dim3(NT),
                       0, stream, (float*)out, (const float*)table,
                       (const long*)tokens, (const long*)positions,
                       (const float*)inv_freq, scale, width);
  else
    hipLaunchKernelGGL(embed_scale_sinpos_kernel<short>, dim3(rows), dim3(NT),
                       0, stream, (float*)out, (const short*)table,
                       (const long*)tokens, (const long*)positions,
                       (const float*)inv_freq, scale, width);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_add_rms_norm_f32res(
    void* residual, const void* d0, long d0_stride, float s0, const void* d1,
    long d1_stride, float s1, const void* weight, float w_offset, float eps,
    void* out, int rows, int width, int is_f32, hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (is_f32)
    hipLaunchKernelGGL((add_rms_norm_f32res_kernel<float, float>), dim3(rows),
                       dim3(NT), 0, stream, (float*)residual,
                       (const float*)d0, d0_stride, s0, (const float*)d1,
                       d1_stride, s1, (const float*)weight, w_offset, eps,
                       (float*)out, width);
  else
    hipLaunchKernelGGL((add_rms_norm_f32res_kernel<short, short>), dim3(rows),
                       dim3(NT), 0, stream, (float*)residual,
                       (const short*)d0, d0_stride, s0, (const short*)d1,
                       d1_stride, s1, (const float*)weight, w_offset, eps,
                       (short*)out, width);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_gated_group_rms_norm(void* out, const void* y,
                                              const void* z, long z_stride,
                                              const void* weight, float eps,
                                              int rows, int inner, int groups,
                                              int is_f32,
                                              hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (groups <= 0 || inner % groups != 0) return hipErrorInvalidValue;
  const int gs = inner / groups;
  if (is_f32)
    hipLaunchKernelGGL((gated_group_rms_norm_kernel<float, float>),
                       dim3(rows, groups), dim3(NT), 0, stream, (float*)out,
                       (const float*)y, (const float*)z, z_stride,
                       (const float*)weight, eps, inner, gs);
  else
    hipLaunchKernelGGL((gated_group_rms_norm_kernel<short, short>),
                       dim3(rows, groups), dim3(NT), 0, stream, (short*)out,
                       (const float*)y, (const short*)z, z_stride,
                       (const float*)weight, eps, inner, gs);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
