// The gated delta rule with a decay per key channel, as a mixer's recurrence, in float32 throughout.
//
// Per head a state S [d, dv]; per token, with unit vectors q (times q_scale) and k of the head's query/key head, values
// v, a step size beta and decays g[i] in (0, 1) per key channel:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          (the read-out sees the token's own write)
// Every column of S runs this on its own, so a lane owns one column, held in registers, and walks the tokens in order.
//
// Three kernels a step: `prepare` turns a token's projections into the recurrence's operands (the short causal
// convolutions with silu, the unit vectors, sigmoid and the decays), `carry` moves the convolutions' last inputs into
// the per-sequence state, `scan` runs the recurrence and `finish` norms the heads' results and gates them.
#include "common.h"
#include "yalm_hip.h"

namespace {

constexpr int GD_THREADS = 256;
constexpr int GD_MAX_TAPS = 16;
constexpr int GD_TOKENS = 16;            // tokens whose operands the scan stages in LDS at a time

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// proj [T, 2 Kq + Vv + H]: q | k | v (before their convolutions) | the step size's logit.
// low [T, H d + H dv]: the decay's and the output gate's pre-activations (the second of each pair of small products).
// prep [T, 2 Kq + Vv + H + H d]: q | k | v | beta | g, ready for the scan.
// conv_w [2 Kq + Vv, taps], the last column is the current token's.  conv_state [n_slots, state_stride] holds, from
// conv_off on, [channel][taps - 1] inputs of the tokens before this step, the latest last.
__global__ __launch_bounds__(GD_THREADS) void gd_prepare_kernel(
    const float* __restrict__ proj, const float* __restrict__ low, const float* __restrict__ conv_w,
    const float* __restrict__ decay_log, const float* __restrict__ decay_bias, const float* __restrict__ state,
    const int* __restrict__ tok_seq, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    float* __restrict__ prep, int H, int Hq, int d, int dv, int taps, float q_scale, float unit_floor, long state_stride,
    long conv_off) {
  extern __shared__ float row[];                  // the token's q | k after convolution and silu
  const int t = blockIdx.x;
  const int Kq = Hq * d, Vv = H * dv, C = 2 * Kq + Vv;
  const int n_in = C + H, n_out = C + H + H * d;
  const int b = tok_seq[t];
  const int slot = seq_slot[b];
  float* out = prep + (size_t)t * n_out;
  if (slot < 0) {                                 // a padding row
    for (int i = threadIdx.x; i < n_out; i += GD_THREADS) out[i] = 0.f;
    return;
  }
  const int p = t - cu_seqlens[b];                // the token's place among its sequence's tokens of this step
  const float* x = proj + (size_t)t * n_in;
  const float* held = state + (size_t)slot * state_stride + conv_off;
  for (int c = threadIdx.x; c < C; c += GD_THREADS) {
    const float* w = conv_w + (size_t)c * taps;
    float acc = w[taps - 1] * x[c];
    for (int back = 1; back < taps; ++back) {
      const float past = back <= p ? proj[(size_t)(t - back) * n_in + c] : held[(size_t)c * (taps - 1) + (taps - 1 - back + p)];
      acc = fmaf(w[taps - 1 - back], past, acc);
    }
    const float a = acc / (1.0f + expf(-acc));
    if (c < 2 * Kq) row[c] = a; else out[c] = a;
  }
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  for (int hh = wave; hh < 2 * Hq; hh += GD_THREADS / WAVE) {         // unit vectors, a head a wave
    const float* r = row + (size_t)hh * d;
    float ss = 0.f;
    for (int i = lane; i < d; i += WAVE) ss = fmaf(r[i], r[i], ss);
    ss = wave_sum(ss);
    const float s = (hh < Hq ? q_scale : 1.0f) / sqrtf(ss + unit_floor);
    for (int i = lane; i < d; i += WAVE) out[(size_t)hh * d + i] = r[i] * s;
  }
  for (int h = threadIdx.x; h < H; h += GD_THREADS) out[C + h] = sigmoidf_(x[C + h]);
  const float* z = low + (size_t)t * (H * d + Vv);
  for (int i = threadIdx.x; i < H * d; i += GD_THREADS)
    out[C + H + i] = expf(-expf(decay_log[i / d]) * softplusf_(z[i] + decay_bias[i]));
}

// The convolutions' inputs that the next step needs: the last taps - 1 of (what was held) ++ (this step's).
__global__ void gd_carry_kernel(const float* __restrict__ proj, float* __restrict__ state,
                                const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot, int C, int n_in,
                                int taps, long state_stride, long conv_off) {
  const int b = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  const int slot = seq_slot[b];
  if (slot < 0 || c >= C) return;
  const int t0 = cu_seqlens[b], n = cu_seqlens[b + 1] - t0, m = taps - 1;
  float* held = state + (size_t)slot * state_stride + conv_off + (size_t)c * m;
  for (int i = 0; i < m; ++i)                     // ascending: what is read lies behind what has been written
    held[i] = n + i < m ? held[n + i] : proj[(size_t)(t0 + n + i - m) * n_in + c];
}

// grid (columns / 64, H, B), one wave: lane j owns column j0 + j of head h of sequence b.
template <int D>
__global__ __launch_bounds__(WAVE) void gd_scan_kernel(const float* __restrict__ prep, float* __restrict__ state,
                                                       const int* __restrict__ cu_seqlens,
                                                       const int* __restrict__ seq_slot, float* __restrict__ raw, int H,
                                                       int Hq, int d, int dv, long state_stride) {
  __shared__ __attribute__((aligned(16))) float sq[GD_TOKENS][D], sk[GD_TOKENS][D], sg[GD_TOKENS][D];
  __shared__ float sv[GD_TOKENS][WAVE], sb[GD_TOKENS];
  const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x, j = blockIdx.x * WAVE + lane;
  const int slot = seq_slot[b];
  if (slot < 0) return;
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (t1 <= t0) return;
  const int Kq = Hq * d, Vv = H * dv, C = 2 * Kq + Vv, n_out = C + H + H * d;
  const int hq = h / (H / Hq);
  const bool live = j < dv;
  float* col = state + (size_t)slot * state_stride + ((size_t)h * d) * dv + (live ? j : 0);
  float S[D];
#pragma unroll
  for (int i = 0; i < D; ++i) S[i] = live && i < d ? col[(size_t)i * dv] : 0.f;
  for (int c0 = t0; c0 < t1; c0 += GD_TOKENS) {
    const int n = min(GD_TOKENS, t1 - c0);
    __syncthreads();
    for (int idx = lane; idx < n * D; idx += WAVE) {
      const int tt = idx / D, i = idx % D;
      const float* r = prep + (size_t)(c0 + tt) * n_out;
      const bool in = i < d;
      sq[tt][i] = in ? r[hq * d + i] : 0.f;
      sk[tt][i] = in ? r[Kq + hq * d + i] : 0.f;
      sg[tt][i] = in ? r[C + H + h * d + i] : 0.f;
    }
    for (int tt = 0; tt < n; ++tt) sv[tt][lane] = live ? prep[(size_t)(c0 + tt) * n_out + 2 * Kq + h * dv + j] : 0.f;
    if (lane < n) sb[lane] = prep[(size_t)(c0 + lane) * n_out + C + h];
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      float kv = 0.f;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        S[i] *= sg[tt][i];
        kv = fmaf(S[i], sk[tt][i], kv);
      }
      const float u = sb[tt] * (sv[tt][lane] - kv);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        S[i] = fmaf(sk[tt][i], u, S[i]);
        o = fmaf(S[i], sq[tt][i], o);
      }
      if (live) raw[(size_t)(c0 + tt) * Vv + h * dv + j] = o;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (i < d) col[(size_t)i * dv] = S[i];
  }
}

// out[t, h dv + j] = raw / rms(raw over the head) * w_norm[j] * sigmoid(gate pre-activation); a wave a (token, head)
template <typename T>
__global__ __launch_bounds__(WAVE) void gd_finish_kernel(const float* __restrict__ raw, const float* __restrict__ low,
                                                         const float* __restrict__ w_norm, const int* __restrict__ tok_seq,
                                                         const int* __restrict__ seq_slot, T* __restrict__ out, int H, int d,
                                                         int dv, float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int Vv = H * dv;
  T* o = out + (size_t)t * Vv + (size_t)h * dv;
  if (seq_slot[tok_seq[t]] < 0) {
    for (int j = lane; j < dv; j += WAVE) o[j] = from_f32<T>(0.f);
    return;
  }
  const float* r = raw + (size_t)t * Vv + (size_t)h * dv;
  const float* z = low + (size_t)t * (H * d + Vv) + (size_t)H * d + (size_t)h * dv;
  float ss = 0.f;
  for (int j = lane; j < dv; j += WAVE) ss = fmaf(r[j], r[j], ss);
  ss = wave_sum(ss);
  const float s = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int j = lane; j < dv; j += WAVE) o[j] = from_f32<T>(r[j] * s * w_norm[j] * sigmoidf_(z[j]));
}

}  // namespace

extern "C" int yalm_gated_delta(const float* proj, const float* low, const float* conv_w, const float* decay_log,
                                const float* decay_bias, const float* w_norm, float* state, float* prep, float* raw,
                                const int* tok_seq, const int* cu_seqlens, const int* seq_slot, void* out, int T, int B,
                                int H, int Hq, int d, int dv, int taps, float q_scale, float unit_floor, float eps,
                                int n_slots, int dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0) return YALM_OK;
  if (H <= 0 || Hq <= 0 || H % Hq != 0 || d <= 0 || d > 256 || dv <= 0 || taps <= 0 || taps > GD_MAX_TAPS || n_slots <= 0 ||
      H > 65535 || B > 65535)
    return YALM_ERR_ARG;
  if (dtype != YALM_F32 && dtype != YALM_BF16) return YALM_ERR_DTYPE;
  const int Kq = Hq * d, C = 2 * Kq + H * dv;
  const long conv_off = (long)H * d * dv, state_stride = conv_off + (long)C * (taps - 1);
  const size_t lds = (size_t)2 * Kq * sizeof(float);
  if (lds > 64 * 1024) return YALM_ERR_ARG;
  gd_prepare_kernel<<<T, GD_THREADS, lds, stream>>>(proj, low, conv_w, decay_log, decay_bias, state, tok_seq, cu_seqlens,
                                                    seq_slot, prep, H, Hq, d, dv, taps, q_scale, unit_floor, state_stride,
                                                    conv_off);
  if (int rc = launch_status(); rc != YALM_OK) return rc;
  if (taps > 1) {
    gd_carry_kernel<<<dim3(ceil_div(C, 256), B), 256, 0, stream>>>(proj, state, cu_seqlens, seq_slot, C, C + H, taps,
                                                                   state_stride, conv_off);
    if (int rc = launch_status(); rc != YALM_OK) return rc;
  }
  const dim3 grid(ceil_div(dv, WAVE), H, B);
#define GD_SCAN(D) gd_scan_kernel<D><<<grid, WAVE, 0, stream>>>(prep, state, cu_seqlens, seq_slot, raw, H, Hq, d, dv, state_stride)
  if (d <= 16) GD_SCAN(16);
  else if (d <= 32) GD_SCAN(32);
  else if (d <= 64) GD_SCAN(64);
  else if (d <= 128) GD_SCAN(128);
  else GD_SCAN(256);
#undef GD_SCAN
  if (int rc = launch_status(); rc != YALM_OK) return rc;
  if (dtype == YALM_F32)
    gd_finish_kernel<float><<<dim3(T, H), WAVE, 0, stream>>>(raw, low, w_norm, tok_seq, seq_slot, (float*)out, H, d, dv, eps);
  else
    gd_finish_kernel<bf16><<<dim3(T, H), WAVE, 0, stream>>>(raw, low, w_norm, tok_seq, seq_slot, (bf16*)out, H, d, dv, eps);
  return launch_status();
}
