// The gated delta rule with a decay per key channel, as a mixer's recurrence, in float32 throughout.
//
// Per head a state S [d, dv]; per token, with unit vectors q (times q_scale) and k of the head's query/key head, values
// v, a step size beta and decays g[i] in (0, 1) per key channel:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          (the read-out sees the token's own write)
// Every column of S runs this on its own, so four lanes own one column, held in registers, and walk the tokens in order.
//
// Four kernels a step: `prepare` turns a token's projections into the recurrence's operands (the short causal
// convolutions with silu, the unit vectors, sigmoid and the decays), `carry` moves the convolutions' last inputs into
// the per-sequence state, `scan` runs the recurrence and `finish` norms the heads' results and gates them.
#include "common.h"
#include "yalm_hip.h"

namespace {

constexpr int GD_THREADS = 256;
constexpr int GD_MAX_TAPS = 16;
// The scan stages the operands of 16 tokens in LDS at a time, or of 4 in steps of single tokens (a quarter of the LDS and
// few registers for what waits: more waves a compute unit, whose loads of the state overlap).

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// proj [T, 2 Kq + Vv + H]: q | k | v (before their convolutions) | the step size's logit.
// low [T, H d + H dv]: the decay's and the output gate's pre-activations (the second of each pair of small products).
// prep [T, 2 Kq + Vv + H + H d]: q | k | v | beta | g, ready for the scan.
// conv_w [2 Kq + Vv, taps], the last column is the current token's.  conv_state [n_slots, state_stride] holds, from
// conv_off on, [channel][taps - 1] inputs of the tokens before this step, the latest last.
// grid (T, 1 .. units): a token's work is cut into units of at most 256 channels so that a step of few tokens still fills
// the chip: unit u < 2 Hq is a query or key head (d <= 256: a thread a channel, the head's sum of squares across the
// workgroup), the next ceil(Vv / 256) units are the values, the last ceil(H d / 256) the decays (the first of them also
// the step sizes).
__global__ __launch_bounds__(GD_THREADS) void gd_prepare_kernel(
    const float* __restrict__ proj, const float* __restrict__ low, const float* __restrict__ conv_w,
    const float* __restrict__ decay_log, const float* __restrict__ decay_bias, const float* __restrict__ state,
    const int* __restrict__ tok_seq, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slot,
    float* __restrict__ prep, int H, int Hq, int d, int dv, int taps, float q_scale, float unit_floor, long state_stride,
    long conv_off) {
  __shared__ float part[2][GD_THREADS / WAVE];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int Kq = Hq * d, Vv = H * dv, C = 2 * Kq + Vv;
  const int n_in = C + H, n_out = C + H + H * d;
  const int v_units = (Vv + GD_THREADS - 1) / GD_THREADS;
  const int units = 2 * Hq + v_units + (H * d + GD_THREADS - 1) / GD_THREADS;
  const int b = tok_seq[t];
  const int slot = seq_slot[b];
  const int p = slot < 0 ? 0 : t - cu_seqlens[b];  // the token's place among its sequence's tokens of this step
  float* out = prep + (size_t)t * n_out;
  const float* x = proj + (size_t)t * n_in;
  const float* held = state + (size_t)max(slot, 0) * state_stride + conv_off;
  // a step of many tokens has workgroups enough: each then walks several units (gridDim.y apart, so heads come before
  // values before decays in every workgroup) and has found its token's sequence once
  for (int unit = blockIdx.y, round = 0; unit < units; unit += gridDim.y, ++round) {
    if (unit >= 2 * Hq + v_units) {               // decays (and step sizes)
      const int du = unit - 2 * Hq - v_units, i = du * GD_THREADS + tid;
      if (du == 0)
        for (int h = tid; h < H; h += GD_THREADS) out[C + h] = slot < 0 ? 0.f : sigmoidf_(x[C + h]);
      if (i < H * d) {
        const float z = low[(size_t)t * (H * d + Vv) + i];
        out[C + H + i] = slot < 0 ? 0.f : expf(-expf(decay_log[i / d]) * softplusf_(z + decay_bias[i]));
      }
      continue;
    }
    const bool head = unit < 2 * Hq;
    const int c = head ? unit * d + tid : 2 * Kq + (unit - 2 * Hq) * GD_THREADS + tid;
    const bool live = head ? tid < d : c < C;
    float a = 0.f;
    if (live && slot >= 0) {
      const float* w = conv_w + (size_t)c * taps;
      float acc = w[taps - 1] * x[c];
      for (int back = 1; back < taps; ++back) {
        const float past = back <= p ? proj[(size_t)(t - back) * n_in + c] : held[(size_t)c * (taps - 1) + (taps - 1 - back + p)];
        acc = fmaf(w[taps - 1 - back], past, acc);
      }
      a = acc / (1.0f + expf(-acc));
    }
    if (!head) {
      if (live) out[c] = a;
      continue;
    }
    // unit vectors: the head's sum of squares across the workgroup (the rounds alternate between two sets of partial
    // sums, and a round's barrier stands between the reads of a set and its next writes)
    float* mine = part[round & 1];
    const float ss = wave_sum(a * a);
    if (tid % WAVE == 0) mine[tid / WAVE] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < GD_THREADS / WAVE; ++w) total += mine[w];
    if (live) out[c] = slot < 0 ? 0.f : a * ((unit < Hq ? q_scale : 1.0f) / sqrtf(total + unit_floor));
  }
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

// grid (columns / GD_COLS, H, B), one wave: lane (c, r) = (lane / GD_ROWS, lane % GD_ROWS) owns the rows r DR .. r DR + DR - 1
// of column j0 + c of head h of sequence b, in registers; the two sums over a column's rows (S^T k and S^T q) are
// finished across the GD_ROWS neighbouring lanes of a column with permutes inside a row of 16 lanes (no LDS).  With
// eight lanes a column a prompt of one sequence keeps dv / 8 waves a head busy and a token costs a lane 4 DR = d / 2
// multiply-adds in a row; with four lanes a column (steps of single tokens) a lane's 16 columns are 64 bytes of a
// state's row, which is what the state's way from and to memory likes.
template <int ROWS>
__device__ __forceinline__ float rows_sum(float x) {
  static_assert(ROWS == 4 || ROWS == 8, "sums over four or eight neighbouring lanes");
  x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));   // lanes 1 0 3 2
  x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));   // lanes 2 3 0 1
  if constexpr (ROWS == 8)                        // every lane of a quad holds the quad's sum: lane 7 - i has the other quad's
    x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));
  return x;
}

template <int DR, int GD_ROWS, int GD_TOKENS>
__global__ __launch_bounds__(WAVE) void gd_scan_kernel(const float* __restrict__ prep, float* __restrict__ state,
                                                       const int* __restrict__ cu_seqlens,
                                                       const int* __restrict__ seq_slot, float* __restrict__ raw, int H,
                                                       int Hq, int d, int dv, long state_stride) {
  static_assert(DR % 4 == 0, "a lane reads its rows' operands four at a time");
  constexpr int GD_COLS = WAVE / GD_ROWS;
  constexpr int LD = DR + 4;             // a row group's operands start 4 banks further on than the one's before
  __shared__ __attribute__((aligned(16))) float sq[GD_TOKENS][GD_ROWS * LD], sk[GD_TOKENS][GD_ROWS * LD],
      sg[GD_TOKENS][GD_ROWS * LD];
  __shared__ float sv[GD_TOKENS][GD_COLS], sb[GD_TOKENS];
  const int b = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
  const int c = lane / GD_ROWS, r = lane % GD_ROWS, j = blockIdx.x * GD_COLS + c;
  const int slot = seq_slot[b];
  if (slot < 0) return;
  const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
  if (t1 <= t0) return;
  const int Kq = Hq * d, Vv = H * dv, C = 2 * Kq + Vv, n_out = C + H + H * d;
  const int hq = h / (H / Hq);
  const bool live = j < dv;
  const int i0 = r * DR;
  float* col = state + (size_t)slot * state_stride + ((size_t)h * d) * dv + (live ? j : 0);
  float S[DR];
#pragma unroll
  for (int i = 0; i < DR; ++i) S[i] = live && i0 + i < d ? col[(size_t)(i0 + i) * dv] : 0.f;
  // The operands of GD_TOKENS tokens wait in LDS; those of the next GD_TOKENS are asked for before the recurrence walks
  // the ones at hand and rest in registers meanwhile, so that memory's latency is paid once a sequence, not once a group.
  constexpr int NLD = GD_TOKENS * GD_ROWS * DR / WAVE, NV = GD_TOKENS * GD_COLS / WAVE;
  static_assert(GD_TOKENS * GD_ROWS * DR % WAVE == 0 && GD_TOKENS * GD_COLS % WAVE == 0 && GD_TOKENS <= WAVE, "whole rounds of loads");
  float pq[NLD], pk[NLD], pg[NLD], pv[NV], pb;
  auto fetch = [&](int c0) {
    const int n = min(GD_TOKENS, t1 - c0);
#pragma unroll
    for (int k = 0; k < NLD; ++k) {
      const int idx = k * WAVE + lane, tt = idx / (GD_ROWS * DR), i = idx % (GD_ROWS * DR);
      const bool in = tt < n && i < d;
      const float* row = prep + (size_t)(c0 + (in ? tt : 0)) * n_out + (in ? i : 0);
      pq[k] = in ? row[hq * d] : 0.f;
      pk[k] = in ? row[Kq + hq * d] : 0.f;
      pg[k] = in ? row[C + H + h * d] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int idx = k * WAVE + lane, tt = idx / GD_COLS, jj = blockIdx.x * GD_COLS + idx % GD_COLS;
      pv[k] = tt < n && jj < dv ? prep[(size_t)(c0 + tt) * n_out + 2 * Kq + h * dv + jj] : 0.f;
    }
    pb = lane < n ? prep[(size_t)(c0 + lane) * n_out + C + h] : 0.f;
  };
  fetch(t0);
  for (int c0 = t0; c0 < t1; c0 += GD_TOKENS) {
    const int n = min(GD_TOKENS, t1 - c0);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NLD; ++k) {
      const int idx = k * WAVE + lane, tt = idx / (GD_ROWS * DR), i = idx % (GD_ROWS * DR);
      const int at = (i / DR) * LD + i % DR;
      sq[tt][at] = pq[k];
      sk[tt][at] = pk[k];
      sg[tt][at] = pg[k];
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int idx = k * WAVE + lane;
      sv[idx / GD_COLS][idx % GD_COLS] = pv[k];
    }
    if (lane < GD_TOKENS) sb[lane] = pb;
    __syncthreads();
    if (c0 + GD_TOKENS < t1) fetch(c0 + GD_TOKENS);
    // A token's operands for this lane's rows come from LDS four at a time (a row group starts on a 16-byte border),
    // and the NEXT token's are asked for before the token at hand is worked: two sets of registers take turns.
    struct Ops {
      float4 g[DR / 4], k[DR / 4], q[DR / 4];
      float beta, v;
    };
    auto take = [&](Ops& o, int tt) {
      const float4* g4 = reinterpret_cast<const float4*>(&sg[tt][r * LD]);
      const float4* k4 = reinterpret_cast<const float4*>(&sk[tt][r * LD]);
      const float4* q4 = reinterpret_cast<const float4*>(&sq[tt][r * LD]);
#pragma unroll
      for (int v = 0; v < DR / 4; ++v) o.g[v] = g4[v], o.k[v] = k4[v], o.q[v] = q4[v];
      o.beta = sb[tt];
      o.v = sv[tt][c];
    };
    auto work = [&](const Ops& o, int tt) {
      float kv0 = 0.f, kv1 = 0.f, kv2 = 0.f, kv3 = 0.f;
#pragma unroll
      for (int v = 0; v < DR / 4; ++v) {
        const float4 g = o.g[v], k = o.k[v];
        const int i = 4 * v;
        S[i] *= g.x, S[i + 1] *= g.y, S[i + 2] *= g.z, S[i + 3] *= g.w;
        kv0 = fmaf(S[i], k.x, kv0);
        kv1 = fmaf(S[i + 1], k.y, kv1);
        kv2 = fmaf(S[i + 2], k.z, kv2);
        kv3 = fmaf(S[i + 3], k.w, kv3);
      }
      const float kv = rows_sum<GD_ROWS>((kv0 + kv1) + (kv2 + kv3));
      const float u = o.beta * (o.v - kv);
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int v = 0; v < DR / 4; ++v) {
        const float4 k = o.k[v], q = o.q[v];
        const int i = 4 * v;
        S[i] = fmaf(k.x, u, S[i]);
        S[i + 1] = fmaf(k.y, u, S[i + 1]);
        S[i + 2] = fmaf(k.z, u, S[i + 2]);
        S[i + 3] = fmaf(k.w, u, S[i + 3]);
        o0 = fmaf(S[i], q.x, o0);
        o1 = fmaf(S[i + 1], q.y, o1);
        o2 = fmaf(S[i + 2], q.z, o2);
        o3 = fmaf(S[i + 3], q.w, o3);
      }
      const float res = rows_sum<GD_ROWS>((o0 + o1) + (o2 + o3));
      if (live && r == 0) raw[(size_t)(c0 + tt) * Vv + h * dv + j] = res;
    };
    Ops A;
    if constexpr (GD_TOKENS <= 4) {                // steps of single tokens: nothing to ask for ahead
      for (int tt = 0; tt < n; ++tt) {
        take(A, tt);
        work(A, tt);
      }
    } else {
      Ops B;
      take(A, 0);
      for (int tt = 0; tt < n; tt += 2) {
        take(B, min(tt + 1, GD_TOKENS - 1));       // rows behind the step's last token hold zeros or older operands: unused
        work(A, tt);
        if (tt + 1 < n) {
          take(A, min(tt + 2, GD_TOKENS - 1));
          work(B, tt + 1);
        }
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DR; ++i)
      if (i0 + i < d) col[(size_t)(i0 + i) * dv] = S[i];
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
  const int units = 2 * Hq + ceil_div(H * dv, GD_THREADS) + ceil_div(H * d, GD_THREADS);
  if (units > 65535 || d > GD_THREADS) return YALM_ERR_ARG;
  // about 16 thousand workgroups at least, none with more units than there are
  const int unit_rows = min(units, max(1, ceil_div(16384, T)));
  gd_prepare_kernel<<<dim3(T, unit_rows), GD_THREADS, 0, stream>>>(proj, low, conv_w, decay_log, decay_bias, state, tok_seq, cu_seqlens,
                                                    seq_slot, prep, H, Hq, d, dv, taps, q_scale, unit_floor, state_stride,
                                                    conv_off);
  if (int rc = launch_status(); rc != YALM_OK) return rc;
  if (taps > 1) {
    gd_carry_kernel<<<dim3(ceil_div(C, 256), B), 256, 0, stream>>>(proj, state, cu_seqlens, seq_slot, C, C + H, taps,
                                                                   state_stride, conv_off);
    if (int rc = launch_status(); rc != YALM_OK) return rc;
  }
  // steps of prompts: eight lanes a column; steps of few tokens a sequence: four
  const bool wide = T >= 32 * B && d > 16;
  const int cols = WAVE / (wide ? 8 : 4);
  if (ceil_div(dv, cols) > 65535) return YALM_ERR_ARG;
  const dim3 grid(ceil_div(dv, cols), H, B);
  const bool few = T <= 4 * B;
#define GD_SCAN_(DR, ROWS, TOKENS) \
  gd_scan_kernel<DR, ROWS, TOKENS><<<grid, WAVE, 0, stream>>>(prep, state, cu_seqlens, seq_slot, raw, H, Hq, d, dv, state_stride)
#define GD_SCAN(DR, ROWS)             \
  do {                                \
    if (few) GD_SCAN_(DR, ROWS, 4);   \
    else GD_SCAN_(DR, ROWS, 16);      \
  } while (0)
  if (wide) {                             // rows a lane: an eighth of the key head, rounded up to the next template
    if (d <= 32) GD_SCAN_(4, 8, 16);          // eight tokens' operands at a time where a lane has many rows: fewer
    else if (d <= 64) GD_SCAN_(8, 8, 16);     // registers wait with the next tokens' operands
    else if (d <= 128) GD_SCAN_(16, 8, 8);
    else GD_SCAN_(32, 8, 8);
  } else {                                // a quarter
    if (d <= 16) GD_SCAN(4, 4);
    else if (d <= 32) GD_SCAN(8, 4);
    else if (d <= 64) GD_SCAN(16, 4);
    else if (d <= 128) GD_SCAN(32, 4);
    else GD_SCAN(64, 4);
  }
#undef GD_SCAN
#undef GD_SCAN_
  if (int rc = launch_status(); rc != YALM_OK) return rc;
  if (dtype == YALM_F32)
    gd_finish_kernel<float><<<dim3(T, H), WAVE, 0, stream>>>(raw, low, w_norm, tok_seq, seq_slot, (float*)out, H, d, dv, eps);
  else
    gd_finish_kernel<bf16><<<dim3(T, H), WAVE, 0, stream>>>(raw, low, w_norm, tok_seq, seq_slot, (bf16*)out, H, d, dv, eps);
  return launch_status();
}
