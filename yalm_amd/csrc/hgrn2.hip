// The gated linear recurrence whose forget gate also decides what is written (HGRN2).  Per head, with the state S
// [d, dv] in float32:
//     q = silu(z_q),  f = l + (1 - l) sigmoid(z_f + b)          (l the gate's lower bound, per head and channel)
//     S <- diag(f) S + (1 - f) v^T,   o = S^T q
// and each head's o is divided by its root mean square over dv and multiplied by a weight shared by the heads.
// Everything behind the projections z_q | z_f | v (float32) is float32.
//
// hgrn2_scan: every column of S runs the recurrence on its own.  A workgroup owns 32 columns of one (sequence, head)
// and walks the sequence's tokens of the step in order; a column is spread over eight lanes, each with NR
// consecutive rows of it in registers (the state is kept column by column, [slot][head][column][row], so that a wave
// reads and writes whole lines of it).  The gates of 16 tokens at a time are formed once by the whole workgroup (from
// projections that were asked for a group ahead and waited in registers) and wait in LDS, where the lanes read them
// four at a time; a lane leaves its share of a column's read-out in LDS and goes on to the next token, and the shares
// of a group's tokens are summed afterwards by all threads at once, so that no token waits for an exchange between
// lanes.  hgrn2_finish: the heads' norm, a wave a (token, head).
#include "common.h"
#include "yalm_hip.h"

namespace {
constexpr int SCAN_THREADS = 256, COL_LANES = 8, SCAN_COLS = SCAN_THREADS / COL_LANES, SCAN_TOKENS = 16;

template <int NR>
__global__ __launch_bounds__(SCAN_THREADS) void hgrn2_scan_kernel(
    const float* __restrict__ proj, const float* __restrict__ f_bias, const float* __restrict__ lower,
    float* __restrict__ state, float* __restrict__ raw, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_slot, int n_heads, int d, int dv) {
  constexpr int DP = NR * COL_LANES;              // rows as the lanes count them (zeros behind d); divides SCAN_THREADS
  constexpr int EL = SCAN_TOKENS * DP / SCAN_THREADS;           // gates a thread forms for a group of tokens
  constexpr int VL = SCAN_TOKENS * SCAN_COLS / SCAN_THREADS;    // values it fetches
  __shared__ float s_q[SCAN_TOKENS][DP];
  __shared__ float s_f[SCAN_TOKENS][DP];
  __shared__ float s_v[SCAN_TOKENS][SCAN_COLS];
  __shared__ float s_part[SCAN_TOKENS][SCAN_THREADS];           // every lane's share of a column's read-out
  const int b = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * SCAN_COLS, tid = threadIdx.x;
  const int col = tid / COL_LANES, rl = tid % COL_LANES, j = c0 + col, r0 = rl * NR;
  const int slot = seq_slot[b];
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  const int Hd = n_heads * d, HV = n_heads * dv, N = 2 * Hd + HV;
  if (slot < 0) {                                 // a padding row: no state is touched, its result is zeros
    for (int t = t0; t < t1; ++t)
      if (rl == 0 && j < dv) raw[(size_t)t * HV + h * dv + j] = 0.f;
    return;
  }
  float* sp = state + (((size_t)slot * n_heads + h) * dv + min(j, dv - 1)) * d;      // this column's rows
  const bool vec = d % 4 == 0 && (((uintptr_t)state) & 15) == 0;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; i += 4) {
    if (vec && r0 + i + 3 < d && j < dv) {
      const float4 v4 = *reinterpret_cast<const float4*>(sp + r0 + i);
      s[i] = v4.x, s[i + 1] = v4.y, s[i + 2] = v4.z, s[i + 3] = v4.w;
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) s[i + k] = (r0 + i + k < d && j < dv) ? sp[r0 + i + k] : 0.f;
    }
  }
  // the thread forms the gates of row gr of the tokens gt, gt + SCAN_THREADS / DP, ... of a group, and fetches the values
  // of column vc of the tokens vt, vt + SCAN_THREADS / SCAN_COLS, ...: always the same row and column
  const int gr = tid % DP, gt = tid / DP, vc = tid % SCAN_COLS, vt = tid / SCAN_COLS;
  const bool row_ok = gr < d, col_ok = c0 + vc < dv;
  const float fb = row_ok ? f_bias[h * d + gr] : 0.f, lo = row_ok ? lower[h * d + gr] : 0.f;
  float zq[EL], zf[EL], zv[VL];
  auto fetch = [&](int tc) {                      // a group's operands into registers: asked for a group ahead
#pragma unroll
    for (int k = 0; k < EL; ++k) {
      const int t = tc + gt + k * (SCAN_THREADS / DP);
      const bool ok = row_ok && t < t1;
      zq[k] = ok ? proj[(size_t)t * N + h * d + gr] : 0.f;
      zf[k] = ok ? proj[(size_t)t * N + Hd + h * d + gr] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < VL; ++k) {
      const int t = tc + vt + k * (SCAN_THREADS / SCAN_COLS);
      zv[k] = col_ok && t < t1 ? proj[(size_t)t * N + 2 * Hd + h * dv + c0 + vc] : 0.f;
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += SCAN_TOKENS) {
    const int n = min(SCAN_TOKENS, t1 - tc);
    __syncthreads();                              // the group before is read
#pragma unroll
    for (int k = 0; k < EL; ++k) {
      const int tt = gt + k * (SCAN_THREADS / DP);
      const float q = zq[k] / (1.0f + expf(-zq[k]));
      const float f = lo + (1.0f - lo) / (1.0f + expf(-(zf[k] + fb)));
      s_q[tt][gr] = row_ok ? q : 0.f;
      s_f[tt][gr] = row_ok ? f : 0.f;
    }
#pragma unroll
    for (int k = 0; k < VL; ++k) s_v[vt + k * (SCAN_THREADS / SCAN_COLS)][vc] = zv[k];
    if (tc + SCAN_TOKENS < t1) fetch(tc + SCAN_TOKENS);
    __syncthreads();
    auto token = [&](int tt) {
      const float v = s_v[tt][col];
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int i = 0; i < NR; i += 4) {
        const float4 f4 = *reinterpret_cast<const float4*>(&s_f[tt][r0 + i]);
        const float4 q4 = *reinterpret_cast<const float4*>(&s_q[tt][r0 + i]);
        s[i] = fmaf(f4.x, s[i] - v, v);           // f S + (1 - f) v
        s[i + 1] = fmaf(f4.y, s[i + 1] - v, v);
        s[i + 2] = fmaf(f4.z, s[i + 2] - v, v);
        s[i + 3] = fmaf(f4.w, s[i + 3] - v, v);
        acc0 = fmaf(s[i], q4.x, acc0);
        acc1 = fmaf(s[i + 1], q4.y, acc1);
        acc0 = fmaf(s[i + 2], q4.z, acc0);
        acc1 = fmaf(s[i + 3], q4.w, acc1);
      }
      s_part[tt][tid] = acc0 + acc1;
    };
    if (n == SCAN_TOKENS) {                       // a whole group: its tokens unrolled, so that a token's reads of LDS stand under the token before
#pragma unroll
      for (int tt = 0; tt < SCAN_TOKENS; ++tt) token(tt);
    } else {
      for (int tt = 0; tt < n; ++tt) token(tt);
    }
    __syncthreads();
    // a column's read-out is the sum over its eight lanes: two (token, column) pairs a thread
#pragma unroll
    for (int k = 0; k < VL; ++k) {
      const int tt = vt + k * (SCAN_THREADS / SCAN_COLS);
      if (tt < n && col_ok) {
        const float4 a = *reinterpret_cast<const float4*>(&s_part[tt][vc * COL_LANES]);
        const float4 c = *reinterpret_cast<const float4*>(&s_part[tt][vc * COL_LANES + 4]);
        raw[(size_t)(tc + tt) * HV + h * dv + c0 + vc] = ((a.x + a.y) + (a.z + a.w)) + ((c.x + c.y) + (c.z + c.w));
      }
    }
  }
  if (j < dv) {
#pragma unroll
    for (int i = 0; i < NR; i += 4) {
      if (vec && r0 + i + 3 < d) {
        *reinterpret_cast<float4*>(sp + r0 + i) = make_float4(s[i], s[i + 1], s[i + 2], s[i + 3]);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (r0 + i + k < d) sp[r0 + i + k] = s[i + k];
      }
    }
  }
}

// out[t, h, :] = raw[t, h, :] / sqrt(mean(raw[t, h, :]^2) + eps) * w; a wave a (token, head)
template <typename T>
__global__ __launch_bounds__(4 * WAVE) void hgrn2_finish_kernel(const float* __restrict__ raw, const float* __restrict__ w,
                                                               T* __restrict__ out, long n_rows, int dv, float eps) {
  const long row = (long)blockIdx.x * 4 + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (row >= n_rows) return;
  const float* src = raw + row * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += WAVE) ss = fmaf(src[i], src[i], ss);
  ss = wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += WAVE) out[row * dv + i] = from_f32<T>(src[i] * f * w[i]);
}
}  // namespace

extern "C" int yalm_hgrn2(const float* proj, const float* f_bias, const float* lower, const float* w_norm, float* state,
                          float* raw, const int* cu_seqlens, const int* seq_slot, void* out, int T, int B, int n_heads,
                          int d, int dv, float eps, int out_dtype, hipStream_t stream) {
  if (T <= 0 || B <= 0) return YALM_OK;
  if (n_heads <= 0 || n_heads > 65535 || d <= 0 || d > 256 || dv <= 0 || ceil_div(dv, SCAN_COLS) > 65535) return YALM_ERR_ARG;
  if (out_dtype != YALM_F32 && out_dtype != YALM_BF16) return YALM_ERR_DTYPE;
  dim3 grid(B, n_heads, ceil_div(dv, SCAN_COLS));
#define YALM_HGRN2_SCAN(NR_)                                                                                          \
  hgrn2_scan_kernel<NR_><<<grid, SCAN_THREADS, 0, stream>>>(proj, f_bias, lower, state, raw, cu_seqlens, seq_slot,    \
                                                            n_heads, d, dv)
  if (d <= 32) YALM_HGRN2_SCAN(4);
  else if (d <= 64) YALM_HGRN2_SCAN(8);
  else if (d <= 128) YALM_HGRN2_SCAN(16);
  else YALM_HGRN2_SCAN(32);
#undef YALM_HGRN2_SCAN
  int rc = launch_status();
  if (rc != YALM_OK) return rc;
  const long n_rows = (long)T * n_heads;
  const int blocks = ceil_div(n_rows, 4);
  if (out_dtype == YALM_F32)
    hgrn2_finish_kernel<float><<<blocks, 4 * WAVE, 0, stream>>>(raw, w_norm, (float*)out, n_rows, dv, eps);
  else
    hgrn2_finish_kernel<bf16><<<blocks, 4 * WAVE, 0, stream>>>(raw, w_norm, (bf16*)out, n_rows, dv, eps);
  return launch_status();
}
