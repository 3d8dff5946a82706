// What stands between the q/k/v product and an attention without rotation: biases, RMS norms over the WHOLE query
// and key projections (all heads at once), a query factor that grows with the position, the blend of the values
// with those an earlier layer made for the same token, and the way into the cache.  A workgroup a token; the row
// waits in LDS between its sums and its results.
//
//   q = (qkv[:Q] + b_q);  q <- q / rms(q) * w_q            (w_q null: no norm)
//   q <- q * (1 + coef ln(floor((p + 1) / every) + 1)) * q_scale      (every 0: no factor)
//   k likewise with w_k (no factor);  v = qkv[Q + K:] + b_v
//   blend 1: v_first <- v;   blend 2: v <- (1 - lam) v + lam v_first      (lam a number on the device)
// head_norm: the norms run a head at a time instead (over the head's d elements, w_q and w_k of d elements shared by
// the heads).  v_from_k: the product has no value part; a head's values are its keys as projected, before their norm
// (dv = d).  rot_dims > 0: behind the norms, of each query and key head's first rot_dims elements the neighbours (2p,
// 2p + 1) are turned by the angle of pair p at the token's position (cos_sin [positions][rot_dims / 2]).
// Heads are written `pad` elements wide (key size d and value size dv may differ; zeros behind): q_out [T, heads,
// pad], keys into their page and the step's staging tile [row][pad], values transposed [pad][row].
#include "common.h"
#include "yalm_hip.h"

namespace {
// a row of a few hundred numbers takes 256 threads, a real model's thousands 1,024 (a decode step has few tokens, and a
// thread's loads wait for each other's results in turn: the fewer rounds the better)
template <typename T, int PACK_THREADS>
__global__ __launch_bounds__(PACK_THREADS) void qkv_pack_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bias, const float* __restrict__ w_q,
    const float* __restrict__ w_k, float eps, float temp_coef, int temp_every, float q_scale, float* __restrict__ v_first,
    int blend, const float* __restrict__ lam_p, T* __restrict__ q_out, T* __restrict__ k_stage, T* __restrict__ v_stage,
    const int* __restrict__ seq_tile0, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, int ring_pages, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const int* __restrict__ seq_slot, const int* __restrict__ seq_len, int n_heads,
    int n_kv_heads, int d, int dv, int pad, int n_pages, int page_layout, T* __restrict__ v_rows, int head_norm,
    int v_from_k, const float2* __restrict__ cos_sin, int rot_dims, int n_positions) {
  extern __shared__ float row[];                  // [Q + K + V], then a factor for every query and key head
  __shared__ float red[PACK_THREADS / WAVE];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int Q = n_heads * d, K = n_kv_heads * d, V = n_kv_heads * dv, N = Q + K + (v_from_k ? 0 : V);
  float* head_f = row + N;                        // head_norm: 1 / rms of each query head, then of each key head
  const float* src = qkv + (size_t)t * N;
  float sq = 0.f, sk = 0.f;
#pragma unroll 4
  for (int i = tid; i < N; i += PACK_THREADS) {
    const float v = src[i] + (bias != nullptr ? bias[i] : 0.f);
    row[i] = v;
    if (i < Q) sq = fmaf(v, v, sq);
    else if (i < Q + K) sk = fmaf(v, v, sk);
  }
  sq = block_sum<PACK_THREADS / WAVE>(sq, red);
  sk = block_sum<PACK_THREADS / WAVE>(sk, red);
  __syncthreads();
  if (head_norm) {                                // a wave a head: the sum of its squares
    for (int hh = tid / WAVE; hh < n_heads + n_kv_heads; hh += PACK_THREADS / WAVE) {
      float s = 0.f;
      for (int e = tid % WAVE; e < d; e += WAVE) s = fmaf(row[hh * d + e], row[hh * d + e], s);
      s = wave_sum(s);
      if (tid % WAVE == 0) head_f[hh] = 1.0f / sqrtf(s / (float)d + eps);
    }
    __syncthreads();
  }
  const int pos = tok_pos[t];
  const float2* cs = rot_dims > 0 ? cos_sin + (size_t)min(max(pos, 0), n_positions - 1) * (rot_dims / 2) : nullptr;
  const int b = tok_seq[t];
  const int slot = b >= 0 ? seq_slot[b] : -1;

  // the queries
  float fq = q_scale;
  if (w_q != nullptr && !head_norm) fq *= 1.0f / sqrtf(sq / (float)Q + eps);
  if (temp_every > 0) fq *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  for (int i = tid; i < n_heads * pad; i += PACK_THREADS) {
    const int h = i / pad, e = i - h * pad;
    float v = 0.f;
    if (e < d) {
      const float f = head_norm && w_q != nullptr ? fq * head_f[h] : fq;
      auto normed = [&](int el) { return row[h * d + el] * f * (w_q != nullptr ? w_q[head_norm ? el : h * d + el] : 1.0f); };
      v = normed(e);
      if (e < rot_dims) {
        const float2 c = cs[e >> 1];
        const float other = normed(e ^ 1);
        v = (e & 1) ? fmaf(v, c.x, other * c.y) : fmaf(v, c.x, -other * c.y);
      }
    }
    q_out[(size_t)t * n_heads * pad + i] = from_f32<T>(v);
  }

  // where this token's key and value go: its page in the cache (a ring keeps the last pages only) and the step's tile
  const int r = pos & (PAGE - 1);
  long page = -1, tile = -1;
  if (slot >= 0 && pos >= 0 && k_pages != nullptr) {
    const int ap = pos / PAGE, last_ap = (seq_len[b] - 1) / PAGE;
    if (ap > last_ap - ring_pages) {
      const int phys = block_table[(size_t)slot * table_stride + (ap % ring_pages)];
      if (phys >= 0 && phys < n_pages) page = phys;
    }
  }
  if (k_stage != nullptr && b >= 0 && pos >= 0) tile = (long)seq_tile0[b] + pos / PAGE;

  const float fk = w_k != nullptr && !head_norm ? 1.0f / sqrtf(sk / (float)K + eps) : 1.0f;
  const float lam = blend == 2 ? lam_p[0] : 0.f;
  for (int i = tid; i < n_kv_heads * pad; i += PACK_THREADS) {
    const int g = i / pad, e = i - g * pad;
    float kv = 0.f, vv = 0.f;
    if (e < d) {
      const float f = head_norm && w_k != nullptr ? head_f[n_heads + g] : fk;
      auto normed = [&](int el) { return row[Q + g * d + el] * f * (w_k != nullptr ? w_k[head_norm ? el : g * d + el] : 1.0f); };
      kv = normed(e);
      if (e < rot_dims) {
        const float2 c = cs[e >> 1];
        const float other = normed(e ^ 1);
        kv = (e & 1) ? fmaf(kv, c.x, other * c.y) : fmaf(kv, c.x, -other * c.y);
      }
    }
    if (e < dv) {
      vv = v_from_k ? row[Q + g * d + e] : row[Q + K + g * dv + e];
      float* first = v_first != nullptr ? v_first + (size_t)t * V + g * dv + e : nullptr;
      if (blend == 1) *first = vv;
      else if (blend == 2) vv = (1.0f - lam) * vv + lam * *first;
    }
    const T kt = from_f32<T>(kv), vt = from_f32<T>(vv);
    // v_rows: the values go there row by row, and a kernel that works a tile of 64 tokens at a time brings them into the
    // transposed places (whole lines instead of two bytes at a time)
    if (v_rows != nullptr) v_rows[(size_t)t * n_kv_heads * pad + i] = vt;
    if (tile >= 0) {
      const size_t base = ((size_t)tile * n_kv_heads + g) * PAGE * pad;
      k_stage[base + (size_t)r * pad + e] = kt;
      if (v_rows == nullptr) v_stage[base + (size_t)e * PAGE + r] = vt;
    }
    if (page >= 0) {
      const size_t base = ((size_t)page * n_kv_heads + g) * PAGE * pad;
      k_pages[base + page_k_offset(page_layout, r, e, pad)] = kt;
      if (v_rows == nullptr) v_pages[base + page_v_offset(page_layout, r, e, pad)] = vt;
    }
  }
}

// The same work a wave a token, the token's row in registers between its sums and its results: no LDS and no barrier
// (a workgroup a token spends most of its time waiting at the barriers of its two sums).  For rows whose parts and heads
// are multiples of four elements (a lane takes four consecutive ones at a time) and at most 256 * NV elements.
template <typename T> struct Pack4;
template <> struct Pack4<float> {
  static __device__ __forceinline__ void store(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
  }
};
template <> struct Pack4<bf16> {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  static __device__ __forceinline__ void store(bf16* p, float a, float b, float c, float d) {
    *reinterpret_cast<bf16x4*>(p) = (bf16x4){static_cast<bf16>(a), static_cast<bf16>(b), static_cast<bf16>(c), static_cast<bf16>(d)};
  }
};
constexpr int PW_WAVES = 4;

// SHAPED: with norms a head, values that are the keys, or the rotation (the other models run the code without them)
template <typename T, int NV, bool SHAPED>
__global__ __launch_bounds__(PW_WAVES * WAVE) void qkv_pack_wave_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bias, const float* __restrict__ w_q,
    const float* __restrict__ w_k, float eps, float temp_coef, int temp_every, float q_scale, float* __restrict__ v_first,
    int blend, const float* __restrict__ lam_p, T* __restrict__ q_out, T* __restrict__ k_stage, T* __restrict__ v_stage,
    const int* __restrict__ seq_tile0, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, int ring_pages, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const int* __restrict__ seq_slot, const int* __restrict__ seq_len, int n_tokens,
    int n_heads, int n_kv_heads, int d, int dv, int pad, int n_pages, int page_layout, T* __restrict__ v_rows,
    int head_norm_, int v_from_k_, const float2* __restrict__ cos_sin, int rot_dims_, int n_positions) {
  // head_norm here: d a power of two from 4 to 256, so that a head's elements lie in d / 4 neighbouring lanes of one round
  const int head_norm = SHAPED ? head_norm_ : 0, v_from_k = SHAPED ? v_from_k_ : 0, rot_dims = SHAPED ? rot_dims_ : 0;
  const int t = blockIdx.x * PW_WAVES + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  if (t >= n_tokens) return;
  const int Q = n_heads * d, K = n_kv_heads * d, V = n_kv_heads * dv, N = Q + K + (v_from_k ? 0 : V);
  const float* src = qkv + (size_t)t * N;
  float4 r[NV], wt[NV];                           // the row and the norm weights of its elements: every load asked for at once
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (j * WAVE + lane) * 4;
    wt[j] = make_float4(1.f, 1.f, 1.f, 1.f);
    if (i < Q && w_q != nullptr) wt[j] = *reinterpret_cast<const float4*>(w_q + (head_norm ? i % d : i));
    else if (i >= Q && i < Q + K && w_k != nullptr) wt[j] = *reinterpret_cast<const float4*>(w_k + (head_norm ? (i - Q) % d : i - Q));
  }

#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (j * WAVE + lane) * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < N) {
      v = *reinterpret_cast<const float4*>(src + i);
      if (bias != nullptr) {
        const float4 b4 = *reinterpret_cast<const float4*>(bias + i);
        v.x += b4.x; v.y += b4.y; v.z += b4.z; v.w += b4.w;
      }
      const float ss = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      if (i < Q) sq += ss;
      else if (i < Q + K) sk += ss;
    }
    r[j] = v;
    if constexpr (SHAPED) {
      if (head_norm) {                            // the sum over the head's lanes (neighbours: exchanges inside their group);
        float ss = i < Q + K ? v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w : 0.f;      // 1 / rms rides on the norm's weights
        for (int o = 1; o < d / 4; o <<= 1) ss += __shfl_xor(ss, o, WAVE);
        const float f = 1.0f / sqrtf(ss / (float)d + eps);
        wt[j].x *= f, wt[j].y *= f, wt[j].z *= f, wt[j].w *= f;
      }
    }
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  const int pos = tok_pos[t];
  const int b = tok_seq[t];
  const int slot = b >= 0 ? seq_slot[b] : -1;
  float fq = q_scale;
  if (w_q != nullptr && !head_norm) fq *= 1.0f / sqrtf(sq / (float)Q + eps);
  if (temp_every > 0) fq *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  const float fk = w_k != nullptr && !head_norm ? 1.0f / sqrtf(sk / (float)K + eps) : 1.0f;
  const float lam = blend == 2 ? lam_p[0] : 0.f;
  const int row = pos & (PAGE - 1);
  const float2* cs = rot_dims > 0 ? cos_sin + (size_t)min(max(pos, 0), n_positions - 1) * (rot_dims / 2) : nullptr;
  // the lane's four elements e .. e + 3 of a head are two of the rotation's pairs
  auto turn = [&](int e, float& a0, float& a1, float& a2, float& a3) {
    if (e < rot_dims) {
      const float2 c = cs[e >> 1];
      const float x = a0 * c.x - a1 * c.y, y = a1 * c.x + a0 * c.y;
      a0 = x, a1 = y;
    }
    if (e + 2 < rot_dims) {
      const float2 c = cs[(e >> 1) + 1];
      const float x = a2 * c.x - a3 * c.y, y = a3 * c.x + a2 * c.y;
      a2 = x, a3 = y;
    }
  };
  long page = -1, tile = -1;
  if (slot >= 0 && pos >= 0 && k_pages != nullptr) {
    const int ap = pos / PAGE, last_ap = (seq_len[b] - 1) / PAGE;
    if (ap > last_ap - ring_pages) {
      const int phys = block_table[(size_t)slot * table_stride + (ap % ring_pages)];
      if (phys >= 0 && phys < n_pages) page = phys;
    }
  }
  if (k_stage != nullptr && b >= 0 && pos >= 0) tile = (long)seq_tile0[b] + pos / PAGE;
  T* qo = q_out + (size_t)t * n_heads * pad;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (j * WAVE + lane) * 4;
    if (i >= N) continue;
    float4 v = r[j];
    if (i < Q) {
      const int h = i / d, e = i - h * d;
      const float4 w4 = wt[j];
      float a0 = v.x * fq * w4.x, a1 = v.y * fq * w4.y, a2 = v.z * fq * w4.z, a3 = v.w * fq * w4.w;
      if constexpr (SHAPED) turn(e, a0, a1, a2, a3);
      Pack4<T>::store(qo + h * pad + e, a0, a1, a2, a3);
    } else if (i < Q + K) {
      const int ik = i - Q, g = ik / d, e = ik - g * d;
      const float4 w4 = wt[j];
      float a0 = v.x * fk * w4.x, a1 = v.y * fk * w4.y, a2 = v.z * fk * w4.z, a3 = v.w * fk * w4.w;
      if constexpr (SHAPED) turn(e, a0, a1, a2, a3);
      if (SHAPED && v_from_k) {                             // the key as projected is the value
        if (v_rows != nullptr) {
          Pack4<T>::store(v_rows + (size_t)t * n_kv_heads * pad + g * pad + e, v.x, v.y, v.z, v.w);
        } else {
          const float vals[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const T vt = from_f32<T>(vals[u]);
            if (tile >= 0) v_stage[((size_t)tile * n_kv_heads + g) * PAGE * pad + (size_t)(e + u) * PAGE + row] = vt;
            if (page >= 0) v_pages[((size_t)page * n_kv_heads + g) * PAGE * pad + page_v_offset(page_layout, row, e + u, pad)] = vt;
          }
        }
      }
      if (tile >= 0) Pack4<T>::store(k_stage + ((size_t)tile * n_kv_heads + g) * PAGE * pad + (size_t)row * pad + e, a0, a1, a2, a3);
      if (page >= 0)                              // four consecutive elements lie together in either layout
        Pack4<T>::store(k_pages + ((size_t)page * n_kv_heads + g) * PAGE * pad + page_k_offset(page_layout, row, e, pad), a0, a1, a2, a3);
    } else {
      const int iv = i - Q - K, g = iv / dv, e = iv - g * dv;
      if (blend == 1) {
        *reinterpret_cast<float4*>(v_first + (size_t)t * V + iv) = v;
      } else if (blend == 2) {
        const float4 f4 = *reinterpret_cast<const float4*>(v_first + (size_t)t * V + iv);
        v.x = (1.0f - lam) * v.x + lam * f4.x; v.y = (1.0f - lam) * v.y + lam * f4.y;
        v.z = (1.0f - lam) * v.z + lam * f4.z; v.w = (1.0f - lam) * v.w + lam * f4.w;
      }
      if (v_rows != nullptr) {
        Pack4<T>::store(v_rows + (size_t)t * n_kv_heads * pad + g * pad + e, v.x, v.y, v.z, v.w);
      } else {
        const float vals[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const T vt = from_f32<T>(vals[u]);
          if (tile >= 0) v_stage[((size_t)tile * n_kv_heads + g) * PAGE * pad + (size_t)(e + u) * PAGE + row] = vt;
          if (page >= 0) v_pages[((size_t)page * n_kv_heads + g) * PAGE * pad + page_v_offset(page_layout, row, e + u, pad)] = vt;
        }
      }
    }
  }
  // the heads' elements behind the key and the value size are zeros
  const T zero = from_f32<T>(0.f);
  if (pad > d) {
    const int extra = pad - d;
    for (int i = lane; i < n_heads * extra; i += WAVE) qo[(i / extra) * pad + d + i % extra] = zero;
    for (int i = lane; i < n_kv_heads * extra; i += WAVE) {
      const int g = i / extra, e = d + i % extra;
      if (tile >= 0) k_stage[((size_t)tile * n_kv_heads + g) * PAGE * pad + (size_t)row * pad + e] = zero;
      if (page >= 0) k_pages[((size_t)page * n_kv_heads + g) * PAGE * pad + page_k_offset(page_layout, row, e, pad)] = zero;
    }
  }
  if (pad > dv) {
    const int extra = pad - dv;
    for (int i = lane; i < n_kv_heads * extra; i += WAVE) {
      const int g = i / extra, e = dv + i % extra;
      if (v_rows != nullptr) {
        v_rows[(size_t)t * n_kv_heads * pad + g * pad + e] = zero;
      } else {
        if (tile >= 0) v_stage[((size_t)tile * n_kv_heads + g) * PAGE * pad + (size_t)e * PAGE + row] = zero;
        if (page >= 0) v_pages[((size_t)page * n_kv_heads + g) * PAGE * pad + page_v_offset(page_layout, row, e, pad)] = zero;
      }
    }
  }
}

// The values of a step of whole prompts from rows [T, G, pad] into the transposed staging tiles and cache pages: a
// workgroup a (tile of 64 tokens, KV head), through LDS, so that every write is a run of consecutive rows.
constexpr int VT_THREADS = 256;
template <typename T>
__global__ __launch_bounds__(VT_THREADS) void v_tiles_kernel(
    const T* __restrict__ v_rows, T* __restrict__ v_stage, T* __restrict__ v_pages, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_tile0, const int* __restrict__ block_table, int table_stride, int ring_pages,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_len, int B, int n_kv_heads, int pad, int n_pages,
    int page_layout) {
  constexpr int VEC = 16 / sizeof(T);             // elements of a 16-byte access (pad is a multiple of 16)
  struct __attribute__((aligned(16))) Chunk { T v[VEC]; };
  extern __shared__ __attribute__((aligned(16))) unsigned char vt_raw[];
  T* tl = reinterpret_cast<T*>(vt_raw);           // [PAGE][pad + VEC]
  const int tile = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (seq_tile0[mid] <= tile) lo = mid; else hi = mid - 1;
  }
  const int b = lo, tq = tile - seq_tile0[b];
  const int start = cu_seqlens[b], len = cu_seqlens[b + 1] - start;
  const int n_rows = min(PAGE, len - tq * PAGE);
  const int row_w = pad + VEC, per_row = pad / VEC;
  for (int i = tid; i < PAGE * per_row; i += VT_THREADS) {
    const int r = i / per_row, c = i - r * per_row;
    Chunk ch;
#pragma unroll
    for (int u = 0; u < VEC; ++u) ch.v[u] = from_f32<T>(0.f);
    if (r < n_rows)
      ch = *reinterpret_cast<const Chunk*>(v_rows + ((size_t)(start + tq * PAGE + r) * n_kv_heads + g) * pad + c * VEC);
    *reinterpret_cast<Chunk*>(tl + r * row_w + c * VEC) = ch;
  }
  __syncthreads();
  T* vp = nullptr;
  const int slot = seq_slot[b];
  if (v_pages != nullptr && slot >= 0 && n_rows > 0) {
    const int last_ap = (seq_len[b] - 1) / PAGE;
    if (tq > last_ap - ring_pages) {
      const int phys = block_table[(size_t)slot * table_stride + (tq % ring_pages)];
      if (phys >= 0 && phys < n_pages) vp = v_pages + ((size_t)phys * n_kv_heads + g) * PAGE * pad;
    }
  }
  T* vs = v_stage + ((size_t)tile * n_kv_heads + g) * PAGE * pad;
  constexpr int RC = PAGE / VEC;                  // runs of VEC consecutive rows in a tile
  for (int i = tid; i < pad * RC; i += VT_THREADS) {
    const int e = i / RC, r0 = (i % RC) * VEC;
    Chunk ch;
#pragma unroll
    for (int u = 0; u < VEC; ++u) ch.v[u] = tl[(r0 + u) * row_w + e];
    *reinterpret_cast<Chunk*>(vs + (size_t)e * PAGE + r0) = ch;      // rows behind the sequence's end are zeros
    // a run of consecutive rows lies together in either page layout; rows behind the end belong to tokens still to
    // come, which write them before anyone reads them
    if (vp != nullptr && r0 < n_rows) *reinterpret_cast<Chunk*>(vp + page_v_offset(page_layout, r0, e, pad)) = ch;
  }
}
}  // namespace

// v_rows `dtype` [T, G, pad] (what yalm_qkv_pack left) into v_stage [n_tiles, G, pad, 64] and the cache pages (null: none).
extern "C" int yalm_v_tiles(const void* v_rows, void* v_stage, void* v_pages, const int* cu_seqlens, const int* seq_tile0,
                            const int* block_table, int table_stride, int ring_pages, const int* seq_slot,
                            const int* seq_len, int B, int n_tiles, int n_kv_heads, int pad, int n_pages, int page_layout,
                            int dtype, hipStream_t stream) {
  if (n_tiles <= 0 || B <= 0) return YALM_OK;
  if (n_kv_heads <= 0 || n_kv_heads > 65535 || pad <= 0 || v_rows == nullptr || v_stage == nullptr ||
      (v_pages != nullptr && (block_table == nullptr || ring_pages <= 0 || seq_len == nullptr)) ||
      !page_layout_ok(page_layout, pad) || (dtype != YALM_F32 && dtype != YALM_BF16))
    return YALM_ERR_ARG;
  if (pad % 16 != 0 || ((((uintptr_t)v_rows) | ((uintptr_t)v_stage) | ((uintptr_t)v_pages)) & 15)) return YALM_ERR_ARG;
  const size_t lds = (size_t)PAGE * (pad + (dtype == YALM_F32 ? 4 : 8)) * (dtype == YALM_F32 ? 4 : 2);
  if (lds > 64 * 1024) return YALM_ERR_ARG;
  dim3 grid(n_tiles, n_kv_heads);
  if (dtype == YALM_F32)
    v_tiles_kernel<float><<<grid, VT_THREADS, lds, stream>>>((const float*)v_rows, (float*)v_stage, (float*)v_pages, cu_seqlens,
                                                             seq_tile0, block_table, table_stride, ring_pages, seq_slot,
                                                             seq_len, B, n_kv_heads, pad, n_pages, page_layout);
  else
    v_tiles_kernel<bf16><<<grid, VT_THREADS, lds, stream>>>((const bf16*)v_rows, (bf16*)v_stage, (bf16*)v_pages, cu_seqlens,
                                                            seq_tile0, block_table, table_stride, ring_pages, seq_slot, seq_len,
                                                            B, n_kv_heads, pad, n_pages, page_layout);
  return launch_status();
}

extern "C" int yalm_qkv_pack(const float* qkv, const float* bias, const float* w_q, const float* w_k, float eps,
                             float temp_coef, int temp_every, float q_scale, float* v_first, int blend,
                             const float* lam, void* q_out, void* k_stage, void* v_stage, const int* seq_tile0,
                             void* k_pages, void* v_pages, const int* block_table, int table_stride, int ring_pages,
                             const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* seq_len, int T,
                             int n_heads, int n_kv_heads, int d, int dv, int pad, int n_pages, int page_layout,
                             int dtype, void* v_rows, int head_norm, int v_from_k, const float* cos_sin, int rot_dims,
                             int n_positions, hipStream_t stream) {
  if (T <= 0) return YALM_OK;
  if ((v_from_k && (d != dv || blend != 0)) || rot_dims < 0 || rot_dims % 2 || rot_dims > d ||
      (rot_dims > 0 && (cos_sin == nullptr || n_positions <= 0)))
    return YALM_ERR_ARG;
  if (n_heads <= 0 || n_kv_heads <= 0 || d <= 0 || dv <= 0 || pad < d || pad < dv || temp_every < 0 || blend < 0 ||
      blend > 2 || (blend != 0 && v_first == nullptr) || (blend == 2 && lam == nullptr) ||
      (k_stage != nullptr && (v_stage == nullptr || seq_tile0 == nullptr)) ||
      (k_pages != nullptr && (v_pages == nullptr || block_table == nullptr || ring_pages <= 0 || seq_len == nullptr)) ||
      !page_layout_ok(page_layout, pad))
    return YALM_ERR_ARG;
  const int n_row = n_heads * d + n_kv_heads * (d + (v_from_k ? 0 : dv));
  const size_t lds = (size_t)(n_row + n_heads + n_kv_heads) * sizeof(float);
  if (lds > 64 * 1024) return YALM_ERR_ARG;
  // a wave a token where a lane can take four elements at a time and the row fits its registers, and where the tokens
  // are many: a few tokens are done sooner by 1,024 threads each (8 tokens of 6,144 numbers: 12 against 25 us)
  const bool heads_fit = !head_norm || (d >= 4 && d <= 256 && (d & (d - 1)) == 0);      // a head in neighbouring lanes
  const bool by_wave = heads_fit && T >= 32 && d % 4 == 0 && dv % 4 == 0 && n_row <= 256 * 32 &&
                       ((((uintptr_t)qkv) | ((uintptr_t)bias) | ((uintptr_t)w_q) | ((uintptr_t)w_k) | ((uintptr_t)v_first) |
                         ((uintptr_t)q_out) | ((uintptr_t)k_stage) | ((uintptr_t)k_pages) | ((uintptr_t)v_rows)) & 15) == 0;
  if (by_wave) {
    const int blocks = ceil_div(T, PW_WAVES);
    const bool shaped = head_norm || v_from_k || rot_dims > 0;
#define YALM_PACK_W(TYPE, NV_)                                                                                           \
  do { if (shaped) YALM_PACK_WS(TYPE, NV_, true); else YALM_PACK_WS(TYPE, NV_, false); } while (0)
#define YALM_PACK_WS(TYPE, NV_, SHAPED_)                                                                                 \
  qkv_pack_wave_kernel<TYPE, NV_, SHAPED_><<<blocks, PW_WAVES * WAVE, 0, stream>>>(                                               \
      qkv, bias, w_q, w_k, eps, temp_coef, temp_every, q_scale, v_first, blend, lam, (TYPE*)q_out, (TYPE*)k_stage,        \
      (TYPE*)v_stage, seq_tile0, (TYPE*)k_pages, (TYPE*)v_pages, block_table, table_stride, ring_pages, tok_seq,         \
      tok_pos, seq_slot, seq_len, T, n_heads, n_kv_heads, d, dv, pad, n_pages, page_layout, (TYPE*)v_rows, head_norm,    \
      v_from_k, (const float2*)cos_sin, rot_dims, n_positions)
#define YALM_PACK_WN(TYPE)                                                                                               \
  if (n_row <= 256 * 4) YALM_PACK_W(TYPE, 4);                                                                            \
  else if (n_row <= 256 * 8) YALM_PACK_W(TYPE, 8);                                                                       \
  else if (n_row <= 256 * 16) YALM_PACK_W(TYPE, 16);                                                                     \
  else if (n_row <= 256 * 24) YALM_PACK_W(TYPE, 24);                                                                     \
  else YALM_PACK_W(TYPE, 32)
    if (dtype == YALM_F32) {
      YALM_PACK_WN(float);
    } else if (dtype == YALM_BF16) {
      YALM_PACK_WN(bf16);
    } else {
      return YALM_ERR_DTYPE;
    }
#undef YALM_PACK_WN
#undef YALM_PACK_W
#undef YALM_PACK_WS
    return launch_status();
  }
  const bool wide = n_row >= 2048;
#define YALM_PACK(TYPE)                                                                                              \
  if (wide) YALM_PACK_N(TYPE, 1024); else YALM_PACK_N(TYPE, 256)
#define YALM_PACK_N(TYPE, NT)                                                                                        \
  qkv_pack_kernel<TYPE, NT><<<T, NT, lds, stream>>>(                                                                 \
      qkv, bias, w_q, w_k, eps, temp_coef, temp_every, q_scale, v_first, blend, lam, (TYPE*)q_out, (TYPE*)k_stage,    \
      (TYPE*)v_stage, seq_tile0, (TYPE*)k_pages, (TYPE*)v_pages, block_table, table_stride, ring_pages, tok_seq,     \
      tok_pos, seq_slot, seq_len, n_heads, n_kv_heads, d, dv, pad, n_pages, page_layout, (TYPE*)v_rows, head_norm,    \
      v_from_k, (const float2*)cos_sin, rot_dims, n_positions)
  if (dtype == YALM_F32) {
    YALM_PACK(float);
  } else if (dtype == YALM_BF16) {
    YALM_PACK(bf16);
  } else {
    return YALM_ERR_DTYPE;
  }
#undef YALM_PACK
#undef YALM_PACK_N
  return launch_status();
}
