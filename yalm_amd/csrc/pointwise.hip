// Small per-row kernels: an embedding with a learned position vector, an activation between the two products of an
// ungated feed-forward (or of a gated one whose products carry biases), the add of a sublayer's result under a gate
// of one number a token, a short causal convolution over time on every channel with its carried inputs, a sigmoid
// gate on an attention's heads, and the way into a walk of looped layers.
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

// out[t, c] = (residual ? h[t, c] : 0) + sum_j w[j, c] in(t - (taps - 1) + j, c) (the weights tap by tap, [taps][D], so
// that neighbouring channels' weights are neighbours): a causal convolution over the tokens
// of a sequence, the last tap on the token itself.  Inputs in front of the step's first token of a sequence come from
// carried[slot][taps - 1][D] (the sequence's last taps - 1 inputs, the newest last; zeros for a new sequence), and a
// padding row (slot -1) reads zeros there.  A thread a (token, channel).
template <typename T, int MAX_TAPS>
__global__ void time_conv_kernel(const T* __restrict__ h, const float* __restrict__ w, const float* __restrict__ carried,
                                 T* __restrict__ out, const int* __restrict__ tok_seq, const int* __restrict__ cu_seqlens,
                                 const int* __restrict__ seq_slot, int D, int taps, int residual) {
  const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= D) return;
  const int b = tok_seq[t];
  const int first = b >= 0 ? cu_seqlens[b] : t, slot = b >= 0 ? seq_slot[b] : -1;
  const int l = t - first;                        // the token's place among its sequence's tokens of this step
  float acc = residual ? to_f32(h[(size_t)t * D + c]) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = l - (taps - 1) + j;
    float v = 0.f;
    if (src >= 0) v = to_f32(h[(size_t)(first + src) * D + c]);
    else if (slot >= 0) v = carried[((size_t)slot * (taps - 1) + (taps - 1 + src)) * D + c];
    acc = fmaf(w[(size_t)j * D + c], v, acc);
  }
  out[(size_t)t * D + c] = from_f32<T>(acc);
}

// The same for VEC consecutive channels a thread (16 bytes of h at a time), D a multiple of VEC.  one_each: every
// sequence brings one token (row t is sequence t), and the thread also moves the carried inputs on: it has read the
// old ones before it writes, and nobody else touches its channels.
template <typename T, int VEC> struct Chunk;
template <> struct Chunk<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Chunk<bf16, 8> {
  typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
  static __device__ __forceinline__ void load(const bf16* p, float* v) {
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = static_cast<float>(x[k]);
  }
  static __device__ __forceinline__ void store(bf16* p, const float* v) {
    bf16x8 x;
#pragma unroll
    for (int k = 0; k < 8; ++k) x[k] = static_cast<bf16>(v[k]);
    *reinterpret_cast<bf16x8*>(p) = x;
  }
};
template <typename E, int VEC>
__global__ void time_conv_vec_kernel(const E* __restrict__ h, const float* __restrict__ w, float* __restrict__ carried,
                                     E* __restrict__ out, const int* __restrict__ tok_seq,
                                     const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, int D, int taps,
                                     int residual, int one_each, int n_tokens, int per_block) {
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
  if (c >= D) return;
  // a workgroup takes per_block tokens that follow each other: a token's earlier inputs are then lines that the
  // same threads have just read
  for (int t = blockIdx.x * per_block; t < min(n_tokens, (int)(blockIdx.x + 1) * per_block); ++t) {
  const int b = one_each ? t : tok_seq[t];
  const int first = one_each ? t : (b >= 0 ? cu_seqlens[b] : t), slot = b >= 0 ? seq_slot[b] : -1;
  const int l = t - first, keep = taps - 1;
  float own[VEC], acc[VEC], v[VEC];
  Chunk<E, VEC>::load(h + (size_t)t * D + c, own);
#pragma unroll
  for (int k = 0; k < VEC; ++k) acc[k] = residual ? own[k] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = l - keep + j;
    if (src >= 0) {
      Chunk<E, VEC>::load(h + (size_t)(first + src) * D + c, v);
    } else if (slot >= 0) {
      const float* row = carried + ((size_t)slot * keep + (keep + src)) * D + c;
#pragma unroll
      for (int k = 0; k < VEC; k += 4) Chunk<float, 4>::load(row + k, v + k);
      if (one_each && j > 0) {                    // the row moves one place towards the oldest
        float* older = carried + ((size_t)slot * keep + (keep + src - 1)) * D + c;
#pragma unroll
        for (int k = 0; k < VEC; k += 4) Chunk<float, 4>::store(older + k, v + k);
      }
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) v[k] = 0.f;
    }
    float wj[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k += 4) Chunk<float, 4>::load(w + (size_t)j * D + c + k, wj + k);
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = fmaf(wj[k], v[k], acc[k]);
  }
  if (one_each && slot >= 0 && keep > 0) {        // the token itself is the newest carried input
    float* newest = carried + ((size_t)slot * keep + (keep - 1)) * D + c;
#pragma unroll
    for (int k = 0; k < VEC; k += 4) Chunk<float, 4>::store(newest + k, own + k);
  }
  Chunk<E, VEC>::store(out + (size_t)t * D + c, acc);
  }
}

// carried[slot] <- the last taps - 1 inputs of each sequence after this step's tokens; a thread a (sequence, channel)
// reads what it needs of the old rows before it writes the new ones
template <typename T, int MAX_TAPS>
__global__ void time_conv_carry_kernel(const T* __restrict__ h, float* __restrict__ carried,
                                       const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, int D,
                                       int taps) {
  const int b = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= D) return;
  const int slot = seq_slot[b];
  if (slot < 0) return;
  const int first = cu_seqlens[b], n = cu_seqlens[b + 1] - first, keep = taps - 1;
  float* rows = carried + (size_t)slot * keep * D + c;
  float fresh[MAX_TAPS];
#pragma unroll
  for (int i = 0; i < MAX_TAPS; ++i) {
    if (i < keep) {
      const int src = n - keep + i;               // place among this step's tokens; negative: an older input
      fresh[i] = src >= 0 ? to_f32(h[(size_t)(first + src) * D + c]) : rows[(size_t)(keep + src) * D];
    }
  }
#pragma unroll
  for (int i = 0; i < MAX_TAPS; ++i)
    if (i < keep) rows[(size_t)i * D] = fresh[i];
}

// out[t, i] = act(z[t, i] + bias[i]) * (z[t, F + i] + bias[F + i]) for i < F: the middle of a gated feed-forward whose
// two first products (gate | up, float32) carry biases; x[t, :] += x_bias (the second product's bias, which that
// product's adding epilogue does not know) on the way.  A workgroup a token, or several where the tokens are few.
template <typename T>
__global__ void gated_bias_act_kernel(const float* __restrict__ z, const float* __restrict__ bias, T* __restrict__ out,
                                      int F, int kind, float* __restrict__ x, const float* __restrict__ x_bias, int D) {
  const int t = blockIdx.x, first = blockIdx.y * blockDim.x + threadIdx.x, stride = gridDim.y * blockDim.x;
  const float* zr = z + (size_t)t * 2 * F;
  for (int i = first; i < F; i += stride) {
    const float v = zr[i] + (bias != nullptr ? bias[i] : 0.f), u = zr[F + i] + (bias != nullptr ? bias[F + i] : 0.f);
    float a;
    if (kind == 0) a = 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
    else if (kind == 1) a = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    else a = v / (1.0f + expf(-v));
    out[(size_t)t * F + i] = from_f32<T>(a * u);
  }
  if (x_bias != nullptr)
    for (int i = first; i < D; i += stride) x[(size_t)t * D + i] += x_bias[i];
}

// o[t, h, e] *= sigmoid(g[t * g_stride + h * dv + e]) for e < dv (heads of o are `pad` wide); a workgroup a token
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ o, const float* __restrict__ g, long g_stride, int n_heads, int dv,
                                    int pad) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < n_heads * dv; i += blockDim.x) {
    const int h = i / dv, e = i - h * dv;
    T* p = o + ((size_t)t * n_heads + h) * pad + e;
    *p = from_f32<T>(to_f32(*p) / (1.0f + expf(-g[(size_t)t * g_stride + i])));
  }
}

// both[t] = [x[t] | x0[t]] in the compute dtype, then x[t] = start: what the product that enters a walk of looped
// layers reads, and what its adding epilogue adds to
template <typename T>
__global__ void loop_pack_kernel(float* __restrict__ x, const float* __restrict__ x0, const float* __restrict__ start,
                                 T* __restrict__ both, int D) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    both[(size_t)t * 2 * D + i] = from_f32<T>(x[(size_t)t * D + i]);
    both[(size_t)t * 2 * D + D + i] = from_f32<T>(x0[(size_t)t * D + i]);
    x[(size_t)t * D + i] = start[i];
  }
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

constexpr int CONV_MAX_TAPS = 16;
extern "C" int yalm_time_conv(const void* h, const float* w, float* carried, void* out, const int* tok_seq,
                              const int* cu_seqlens, const int* seq_slot, int T, int B, int D, int taps, int residual,
                              int one_each, int dtype, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (one_each && T != B) return YALM_ERR_ARG;
  if (D <= 0 || B <= 0 || taps <= 0 || taps > CONV_MAX_TAPS || h == out ||
      (taps > 1 && carried == nullptr) || ceil_div(D, 256) > 65535)
    return YALM_ERR_ARG;
  const int vec = dtype == YALM_F32 ? 4 : 8;
  if (D % vec == 0 && (((uintptr_t)h | (uintptr_t)out | (uintptr_t)carried) & 15) == 0 && (dtype == YALM_F32 || dtype == YALM_BF16)) {
    const int lanes = D / vec, vthreads = lanes >= 256 ? 256 : 64;
    const int per_block = (long)T * D >= 2048L * 4096 ? 4 : 1;      // measured: 20.1 -> 15.8 us at 2,048 x 4,096, no gain below
    dim3 vgrid(ceil_div(T, per_block), ceil_div(lanes, vthreads)), vcgrid(B, ceil_div(D, 256));
    if (dtype == YALM_F32) {
      time_conv_vec_kernel<float, 4><<<vgrid, vthreads, 0, stream>>>((const float*)h, w, carried, (float*)out, tok_seq, cu_seqlens,
                                                                    seq_slot, D, taps, residual, one_each, T, per_block);
      if (taps > 1 && !one_each)
        time_conv_carry_kernel<float, CONV_MAX_TAPS><<<vcgrid, 256, 0, stream>>>((const float*)h, carried, cu_seqlens, seq_slot, D, taps);
    } else {
      time_conv_vec_kernel<bf16, 8><<<vgrid, vthreads, 0, stream>>>((const bf16*)h, w, carried, (bf16*)out, tok_seq, cu_seqlens,
                                                                   seq_slot, D, taps, residual, one_each, T, per_block);
      if (taps > 1 && !one_each)
        time_conv_carry_kernel<bf16, CONV_MAX_TAPS><<<vcgrid, 256, 0, stream>>>((const bf16*)h, carried, cu_seqlens, seq_slot, D, taps);
    }
    return launch_status();
  }
  const int threads = D >= 256 ? 256 : 64;
  dim3 grid(T, ceil_div(D, threads)), cgrid(B, ceil_div(D, threads));
  if (dtype == YALM_F32) {
    time_conv_kernel<float, CONV_MAX_TAPS><<<grid, threads, 0, stream>>>((const float*)h, w, carried, (float*)out, tok_seq,
                                                                         cu_seqlens, seq_slot, D, taps, residual);
    if (taps > 1)
      time_conv_carry_kernel<float, CONV_MAX_TAPS><<<cgrid, threads, 0, stream>>>((const float*)h, carried, cu_seqlens, seq_slot, D, taps);
  } else if (dtype == YALM_BF16) {
    time_conv_kernel<bf16, CONV_MAX_TAPS><<<grid, threads, 0, stream>>>((const bf16*)h, w, carried, (bf16*)out, tok_seq,
                                                                        cu_seqlens, seq_slot, D, taps, residual);
    if (taps > 1)
      time_conv_carry_kernel<bf16, CONV_MAX_TAPS><<<cgrid, threads, 0, stream>>>((const bf16*)h, carried, cu_seqlens, seq_slot, D, taps);
  } else {
    return YALM_ERR_DTYPE;
  }
  return launch_status();
}

extern "C" int yalm_gated_bias_act(const float* z, const float* bias, void* out, int T, int F, int kind, int out_dtype,
                                   float* x, const float* x_bias, int D, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (F <= 0 || kind < 0 || kind > 2 || (x_bias != nullptr && (x == nullptr || D <= 0))) return YALM_ERR_ARG;
  const int threads = 256;
  int slices = T >= 512 ? 1 : ceil_div(512, T);                   // a step of few tokens still fills the chip
  slices = slices < ceil_div(F, threads) ? slices : ceil_div(F, threads);
  dim3 grid(T, slices > 0 ? slices : 1);
  if (out_dtype == YALM_F32)
    gated_bias_act_kernel<float><<<grid, threads, 0, stream>>>(z, bias, (float*)out, F, kind, x, x_bias, D);
  else if (out_dtype == YALM_BF16)
    gated_bias_act_kernel<bf16><<<grid, threads, 0, stream>>>(z, bias, (bf16*)out, F, kind, x, x_bias, D);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_sigmoid_gate(void* o, const float* g, long g_stride, int T, int n_heads, int dv, int pad, int dtype,
                                 hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (n_heads <= 0 || dv <= 0 || pad < dv || g_stride < (long)n_heads * dv) return YALM_ERR_ARG;
  const int threads = n_heads * dv >= 2048 ? 1024 : 256;
  if (dtype == YALM_F32)
    sigmoid_gate_kernel<float><<<T, threads, 0, stream>>>((float*)o, g, g_stride, n_heads, dv, pad);
  else if (dtype == YALM_BF16)
    sigmoid_gate_kernel<bf16><<<T, threads, 0, stream>>>((bf16*)o, g, g_stride, n_heads, dv, pad);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}

extern "C" int yalm_loop_pack(float* x, const float* x0, const float* start, void* both, int T, int D, int dtype,
                              hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if (D <= 0) return YALM_ERR_ARG;
  const int threads = D >= 2048 ? 1024 : 256;
  if (dtype == YALM_F32)
    loop_pack_kernel<float><<<T, threads, 0, stream>>>(x, x0, start, (float*)both, D);
  else if (dtype == YALM_BF16)
    loop_pack_kernel<bf16><<<T, threads, 0, stream>>>(x, x0, start, (bf16*)both, D);
  else
    return YALM_ERR_DTYPE;
  return launch_status();
}
