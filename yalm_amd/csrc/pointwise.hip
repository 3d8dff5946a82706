// Small per-row kernels: an embedding with a learned position vector, an activation between the two products of an
// ungated feed-forward, and the add of a sublayer's result under a gate of one number a token.
#include "common.h"
#include "yalm_hip.h"

namespace {

// x[t, :] = table[tokens[t], :] * scale + positions_table[positions[t], :]
template <typename T>
__global__ void embed_learned_kernel(const T* __restrict__ table, const T* __restrict__ pos_table,
                                     const int* __restrict__ tokens, const int* __restrict__ positions, float scale,
                                     float* __restrict__ out, int D, int V, int P) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  float* o = out + (size_t)t * D;
  if (tok < 0 || tok >= V) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = 0.f;
    return;
  }
  const T* row = table + (size_t)tok * D;
  const T* pr = pos_table + (size_t)min(max(positions[t], 0), P - 1) * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = fmaf(to_f32(row[i]), scale, to_f32(pr[i]));
}

// activation codes: 0 the gelu with the error function, z/2 (1 + erf(z / sqrt(2))); 1 its tanh form; 2 silu
template <typename T>
__global__ void activate_kernel(const float* __restrict__ z, T* __restrict__ out, long n, int kind) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = z[i];
    float a;
    if (kind == 0) a = 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
    else if (kind == 1) a = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    else a = v / (1.0f + expf(-v));
    out[i] = from_f32<T>(a);
  }
}

// x[t, :] += sigmoid(h[t, :] . w) * y[t, :]; a block a token
template <typename T, int NW>
__global__ __launch_bounds__(NW * WAVE) void gated_add_kernel(const float* __restrict__ y, const T* __restrict__ h, const T* __restrict__ w,
                                 float* __restrict__ x, int D, int accumulate) {
  __shared__ float red[NW];
  const int t = blockIdx.x;
  const T* hr = h + (size_t)t * D;
  float dot = 0.f;
  for (int i = threadIdx.x; i < D; i += NW * WAVE) dot = fmaf(to_f32(hr[i]), to_f32(w[i]), dot);
  dot = block_sum<NW>(dot, red);
  const float s = 1.0f / (1.0f + expf(-dot));
  const float* yr = y + (size_t)t * D;
  float* xr = x + (size_t)t * D;
  for (int i = threadIdx.x; i < D; i += NW * WAVE) xr[i] = accumulate ? fmaf(s, yr[i], xr[i]) : s * yr[i];
}

}  // namespace

extern "C" int yalm_embed_learned(const void* table, const void* pos_table, int dtype, const int* tokens,
                                  const int* positions, float scale, float* out, int T, int D, int V, int P,
                                  hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0 || V <= 0 || P <= 0) return YALM_ERR_ARG;
  const int threads = D >= 1024 ? 1024 : (D >= 256 ? 256 : 64);
  if (dtype == YALM_F32)
    embed_learned_kernel<float><<<T, threads, 0, stream>>>((const float*)table, (const float*)pos_table, tokens, positions,
                                                           scale, out, D, V, P);
  else if (dtype == YALM_BF16)
    embed_learned_kernel<bf16><<<T, threads, 0, stream>>>((const bf16*)table, (const bf16*)pos_table, tokens, positions,
                                                          scale, out, D, V, P);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_activate(const float* z, void* out, long n, int kind, int out_dtype, hipStream_t stream) {
  if (n <= 0) return YALM_OK;
  if (kind < 0 || kind > 2) return YALM_ERR_ARG;
  const int blocks = (int)((n + 1023) / 1024 < 8192 ? (n + 1023) / 1024 : 8192);
  if (out_dtype == YALM_F32)
    activate_kernel<float><<<blocks, 256, 0, stream>>>(z, (float*)out, n, kind);
  else if (out_dtype == YALM_BF16)
    activate_kernel<bf16><<<blocks, 256, 0, stream>>>(z, (bf16*)out, n, kind);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_gated_add(const float* y, const void* h, const void* w, int dtype, float* x, int T, int D,
                              int accumulate, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0) return YALM_ERR_ARG;
  // a step of few tokens has few workgroups: sixteen waves a token then, four otherwise
  const bool wide = D >= 2048 && T <= 256;
  if (dtype == YALM_F32) {
    if (wide) gated_add_kernel<float, 16><<<T, 1024, 0, stream>>>(y, (const float*)h, (const float*)w, x, D, accumulate);
    else gated_add_kernel<float, 4><<<T, 256, 0, stream>>>(y, (const float*)h, (const float*)w, x, D, accumulate);
  } else if (dtype == YALM_BF16) {
    if (wide) gated_add_kernel<bf16, 16><<<T, 1024, 0, stream>>>(y, (const bf16*)h, (const bf16*)w, x, D, accumulate);
    else gated_add_kernel<bf16, 4><<<T, 256, 0, stream>>>(y, (const bf16*)h, (const bf16*)w, x, D, accumulate);
  } else {
    return YALM_ERR_DTYPE;
  }
  return launch_status();
}
