// Softmax attention against the paged KV cache with scores and weights kept
// in fp32 end to end, for any (query/key dim, value dim, group size).
//
//  * qk_norm_temp_cache: per token, RMS-normalise the WHOLE query projection
//    (all heads at once) and the whole key projection with plain weights,
//    scale the query by a position-dependent temperature
//        1 + coef * ln(floor((pos + 1) / every) + 1),
//    write q (fp32) out and scatter k / v into the paged cache.
//  * ctx_attention_f32: causal attention of a flat variable-length query
//    batch against each sequence's pages (the portion's own keys are already
//    in the cache). Queries of one block share a kv head: in prefill a block
//    takes 16 consecutive tokens of one query head, in decode it takes the
//    query heads of one group so the group's K/V tile is staged once.
//    K/V tiles of 64 keys are converted to fp32 in LDS; a lane owns one key
//    for the score and softmax phase and one output column per 64 for the
//    weighted sum. An optional per-(token, head) gate multiplies the result
//    by sigmoid(gate) before it is stored.
#include "dtype_io.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;
constexpr int ROWS = 16;          // query rows per block
constexpr int RPW = ROWS / NW;    // rows per wave
constexpr int BK = 64;            // keys per tile (lane <-> key)
constexpr int MAX_DV = 256;
constexpr int NVC = MAX_DV / 64;  // output columns per lane

template <typename T>
__global__ void qk_norm_temp_cache_kernel(
    float* __restrict__ q_out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, long row_stride, const float* __restrict__ qw,
    const float* __restrict__ kw, const long* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ k_cache,
    T* __restrict__ v_cache, float eps, float temp_coef, int temp_every,
    int q_width, int kv_heads, int D, int DV, int block_size) {
  __shared__ float scratch[NW];
  const long t = blockIdx.x;
  const T* qr = q + t * row_stride;
  const T* kr = k + t * row_stride;
  const T* vr = v + t * row_stride;
  const int k_width = kv_heads * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_width; i += NT) {
    const float x = ld_f32(qr, i);
    ss += x * x;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  float qinv = 1.0f / sqrtf(ss / (float)q_width + eps);
  const long pos = positions[t];
  if (temp_every > 0)
    qinv *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  for (int i = threadIdx.x; i < q_width; i += NT)
    q_out[t * q_width + i] = ld_f32(qr, i) * qw[i] * qinv;

  ss = 0.f;
  for (int i = threadIdx.x; i < k_width; i += NT) {
    const float x = ld_f32(kr, i);
    ss += x * x;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float kinv = 1.0f / sqrtf(ss / (float)k_width + eps);
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  const long blk = slot / block_size, off = slot % block_size;
  for (int i = threadIdx.x; i < k_width; i += NT) {
    const int g = i / D, d = i % D;
    st_f32(k_cache, ((blk * kv_heads + g) * block_size + off) * D + d,
           ld_f32(kr, i) * kw[i] * kinv);
  }
  for (int i = threadIdx.x; i < kv_heads * DV; i += NT) {
    const int g = i / DV, d = i % DV;
    v_cache[((blk * kv_heads + g) * block_size + off) * DV + d] = vr[i];
  }
}

template <typename T>
__global__ void __launch_bounds__(NT) ctx_attention_f32_kernel(
    T* __restrict__ out, const float* __restrict__ q,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    const T* __restrict__ gate, long gate_stride, float scale, int heads,
    int kv_heads, int D, int DV, int block_size, int hpb) {
  extern __shared__ float lds[];
  const int s = blockIdx.y;
  const int q0 = cu_q[s];
  const int q_len = cu_q[s + 1] - q0;
  const int tpb = ROWS / hpb;  // tokens per block
  const int tok0 = blockIdx.x * tpb;
  if (tok0 >= q_len) return;
  const int head0 = blockIdx.z * hpb;
  const int g = head0 / (heads / kv_heads);
  const int ctx = ctx_lens[s];
  const int ntok = min(tpb, q_len - tok0);
  const int nrows = ntok * hpb;
  // absolute position of the block's last query bounds the keys it needs
  const int last_pos = ctx - q_len + tok0 + ntok - 1;

  const int KS = D + 1;  // padded K row: lane-per-key reads hit distinct banks
  float* Ks = lds;                   // [BK][D+1]
  float* Vs = Ks + BK * KS;          // [BK][DV]
  float* Qs = Vs + BK * DV;          // [D][ROWS] (transposed)
  float* Ps = Qs + D * ROWS;         // [NW][BK][RPW]

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;

  // stage the block's queries, pre-multiplied by the softmax scale
  for (int e = threadIdx.x; e < ROWS * D; e += NT) {
    const int r = e / D, d = e % D;
    float v = 0.f;
    if (r < nrows) {
      const int tok = q0 + tok0 + r / hpb, hd = head0 + r % hpb;
      v = q[((long)tok * heads + hd) * D + d] * scale;
    }
    Qs[d * ROWS + r] = v;
  }

  float m[RPW], l[RPW], acc[RPW][NVC];
  int qpos[RPW];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
    const int r = wave * RPW + i;
    qpos[i] = r < nrows ? ctx - q_len + tok0 + r / hpb : -1;
#pragma unroll
    for (int c = 0; c < NVC; ++c) acc[i][c] = 0.f;
  }
  const int* bt = block_tables + (long)s * bt_stride;

  for (int k0 = 0; k0 <= last_pos; k0 += BK) {
    __syncthreads();  // previous tile fully consumed (and Qs visible)
    const int nk = min(BK, last_pos + 1 - k0);
    for (int e = threadIdx.x; e < BK * D; e += NT) {
      const int j = e / D, d = e % D;
      float v = 0.f;
      if (j < nk) {
        const int kp = k0 + j;
        const long blk = bt[kp / block_size];
        v = ld_f32(k_cache,
                   ((blk * kv_heads + g) * block_size + kp % block_size) * D + d);
      }
      Ks[j * KS + d] = v;
    }
    for (int e = threadIdx.x; e < BK * DV; e += NT) {
      const int j = e / DV, d = e % DV;
      float v = 0.f;
      if (j < nk) {
        const int kp = k0 + j;
        const long blk = bt[kp / block_size];
        v = ld_f32(v_cache,
                   ((blk * kv_heads + g) * block_size + kp % block_size) * DV + d);
      }
      Vs[j * DV + d] = v;
    }
    __syncthreads();

    // scores: lane = key, RPW rows of this wave at once
    float sc[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) sc[i] = 0.f;
    const float* krow = Ks + lane * KS;
    const float* qcol = Qs + wave * RPW;
    for (int d = 0; d < D; ++d) {
      const float kv = krow[d];
#pragma unroll
      for (int i = 0; i < RPW; ++i) sc[i] += qcol[d * ROWS + i] * kv;
    }
    const int kp = k0 + lane;
    float* pw = Ps + wave * BK * RPW;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      const bool vis = kp <= qpos[i];
      const float sv = vis ? sc[i] : -INFINITY;
      const float mt = wave_reduce_max(sv);
      const float mn = fmaxf(m[i], mt);
      // a row with no visible key in this tile keeps mn = -inf only while
      // it has seen nothing at all; guard the exp arguments
      const float corr = (mn == -INFINITY) ? 1.f : expf(m[i] - mn);
      const float pv = vis ? expf(sv - mn) : 0.f;
      l[i] = l[i] * corr + wave_reduce_sum(pv);
      m[i] = mn;
#pragma unroll
      for (int c = 0; c < NVC; ++c) acc[i][c] *= corr;
      pw[lane * RPW + i] = pv;
    }
    // weighted sum: lane = output column (+64 c); weights broadcast from LDS
    // (each wave reads only what it wrote: no block barrier needed)
    for (int j = 0; j < nk; ++j) {
      float pj[RPW];
#pragma unroll
      for (int i = 0; i < RPW; ++i) pj[i] = pw[j * RPW + i];
#pragma unroll
      for (int c = 0; c < NVC; ++c) {
        const int col = lane + 64 * c;
        if (col < DV) {
          const float vv = Vs[j * DV + col];
#pragma unroll
          for (int i = 0; i < RPW; ++i) acc[i][c] += pj[i] * vv;
        }
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int r = wave * RPW + i;
    if (r >= nrows) continue;
    const int tok = q0 + tok0 + r / hpb, hd = head0 + r % hpb;
    float f = 1.0f / l[i];
    if (gate) {
      const float gv = ld_f32(gate, (long)tok * gate_stride + hd);
      f *= 1.0f / (1.0f + expf(-gv));
    }
#pragma unroll
    for (int c = 0; c < NVC; ++c) {
      const int col = lane + 64 * c;
      if (col < DV) st_f32(out, ((long)tok * heads + hd) * DV + col, acc[i][c] * f);
    }
  }
}

}  // namespace

extern "C" hipError_t ks_qk_norm_temp_cache(
    void* q_out, const void* q, const void* k, const void* v, long row_stride,
    const void* qw, const void* kw, const void* positions,
    const void* slot_mapping, void* k_cache, void* v_cache, float eps,
    float temp_coef, int temp_every, int tokens, int heads, int kv_heads,
    int D, int DV, int block_size, int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (is_f32)
    hipLaunchKernelGGL(qk_norm_temp_cache_kernel<float>, dim3(tokens), dim3(NT),
                       0, stream, (float*)q_out, (const float*)q,
                       (const float*)k, (const float*)v, row_stride,
                       (const float*)qw, (const float*)kw,
                       (const long*)positions, (const int*)slot_mapping,
                       (float*)k_cache, (float*)v_cache, eps, temp_coef,
                       temp_every, heads * D, kv_heads, D, DV, block_size);
  else
    hipLaunchKernelGGL(qk_norm_temp_cache_kernel<short>, dim3(tokens), dim3(NT),
                       0, stream, (float*)q_out, (const short*)q,
                       (const short*)k, (const short*)v, row_stride,
                       (const float*)qw, (const float*)kw,
                       (const long*)positions, (const int*)slot_mapping,
                       (short*)k_cache, (short*)v_cache, eps, temp_coef,
                       temp_every, heads * D, kv_heads, D, DV, block_size);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_ctx_attention_f32(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const void* block_tables, int bt_stride, const void* cu_q,
    const void* ctx_lens, const void* gate, long gate_stride, float scale,
    int num_seqs, int max_q_len, int heads, int kv_heads, int D, int DV,
    int block_size, int is_f32, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return hipSuccess;
  if (DV > MAX_DV || D < 1 || kv_heads < 1 || heads % kv_heads != 0)
    return hipErrorInvalidValue;
  // decode: one token per sequence, so a block takes heads of one group
  int hpb = 1;
  if (max_q_len == 1) {
    const int gs = heads / kv_heads;
    for (int c = 1; c <= ROWS && c <= gs; ++c)
      if (gs % c == 0) hpb = c;
  }
  const int tpb = ROWS / hpb;
  const size_t smem =
      sizeof(float) * ((size_t)BK * (D + 1) + (size_t)BK * DV +
                       (size_t)D * ROWS + (size_t)NW * BK * RPW);
  if (smem > 160 * 1024) return hipErrorInvalidValue;
  dim3 grid(cdiv(max_q_len, tpb), num_seqs, heads / hpb);
  hipError_t e;
  if (is_f32) {
    auto fn = ctx_attention_f32_kernel<float>;
    if (smem > 48 * 1024) {
      e = hipFuncSetAttribute((const void*)fn,
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)smem);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(fn, grid, dim3(NT), smem, stream, (float*)out,
                       (const float*)q, (const float*)k_cache,
                       (const float*)v_cache, (const int*)block_tables,
                       bt_stride, (const int*)cu_q, (const int*)ctx_lens,
                       (const float*)gate, gate_stride, scale, heads, kv_heads,
                       D, DV, block_size, hpb);
  } else {
    auto fn = ctx_attention_f32_kernel<short>;
    if (smem > 48 * 1024) {
      e = hipFuncSetAttribute((const void*)fn,
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)smem);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(fn, grid, dim3(NT), smem, stream, (short*)out,
                       (const float*)q, (const short*)k_cache,
                       (const short*)v_cache, (const int*)block_tables,
                       bt_stride, (const int*)cu_q, (const int*)ctx_lens,
                       (const short*)gate, gate_stride, scale, heads, kv_heads,
                       D, DV, block_size, hpb);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
