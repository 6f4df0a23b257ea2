// Short causal convolutions over time with a state per sequence, and the gated delta rule.
//
// Short convolution: y_t[c] = sum_j w[c][j] * u_(t - taps + 1 + j)[c], zeros before a sequence's first token. The
// last taps - 1 inputs u of a sequence live in its state slot `[slots][taps - 1][C]` (the newest last), so a
// sequence may be cut into steps anywhere. The kernels that convolve read the state; `conv_state_update` writes it
// in a launch of its own behind them, so no reader meets a writer.
//
// Gated delta rule, per value head with state S `[key_dim][value_dim]` (float32, in the sequence's slot):
//   S <- diag(g) S ;  u = beta (v - S^T k) ;  S <- S + k u^T ;  o = S^T q
// with q and k unit vectors (q also times key_dim^(-1/2)), beta in (0, 1) and one decay in (0, 1) per head and
// key channel. `delta_prepare` makes q, k, v, beta and g of every token of a step, in parallel over tokens;
// `gated_delta_scan` walks each sequence's tokens in order.
#include "common.h"

#define CONV_MAX_TAPS 8

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// The convolution's sum for row t (of the sequence that starts at row `start`), channel c of the C convolved
// columns, whose inputs are columns of `u` rows `row` apart.
__device__ __forceinline__ float conv_at(const float* __restrict__ u, size_t row, const float* __restrict__ w,
                                         const float* __restrict__ hist, int taps, int C, int t, int start, int c) {
  float y = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = t - (taps - 1) + j;
    // before the step's first row of the sequence: the state, whose entry i is the input of row start - (taps-1) + i
    const float v = src >= start ? u[static_cast<size_t>(src) * row + c]
                                 : hist[static_cast<size_t>(src - start + taps - 1) * C + c];
    y = fmaf(w[c * taps + j], v, y);
  }
  return y;
}

// ---------------------------------------------------------------- q, k, v of an attention with short convolutions
// Row t of `u` holds [q (nq) | k (nk) | v (nv)] as projected (C = nq + nk + nv columns are convolved). out row:
// the same columns convolved; then, where wq / wk are given, q and k each divided by the root mean square over
// their whole width (all heads together; mean over `count_q` / `count_k` values, which may be fewer than the
// columns where heads carry padding columns of zeros) and multiplied by their weights.
__global__ void conv_qkv_kernel(const float* __restrict__ u, int row, const float* __restrict__ w, int taps,
                                const float* __restrict__ state, const int* __restrict__ state_slots,
                                const int* __restrict__ seq_of_row, const int* __restrict__ query_start,
                                int nq, int nk, int nv, const float* __restrict__ wq, const float* __restrict__ wk,
                                float count_q, float count_k, float eps, float* __restrict__ out, int out_row) {
  extern __shared__ float vals[];
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int s = seq_of_row[t];
  const int start = query_start[s];
  const int C = nq + nk + nv;
  const float* hist = state + static_cast<size_t>(state_slots[s]) * (taps - 1) * C;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const float y = taps > 1 ? conv_at(u, row, w, hist, taps, C, t, start, c)
                             : w[c] * u[static_cast<size_t>(t) * row + c];
    vals[c] = y;
    if (c < nq) sq = fmaf(y, y, sq);
    else if (c < nq + nk) sk = fmaf(y, y, sk);
  }
  float iq = 1.f, ik = 1.f;
  if (wq) iq = 1.0f / sqrtf(block_sum(sq, scratch) / count_q + eps);
  if (wk) ik = 1.0f / sqrtf(block_sum(sk, scratch) / count_k + eps);
  __syncthreads();
  float* o = out + static_cast<size_t>(t) * out_row;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float y = vals[c];
    if (c < nq) { if (wq) y = (y * iq) * wq[c]; }
    else if (c < nq + nk) { if (wk) y = (y * ik) * wk[c - nq]; }
    o[c] = y;
  }
}

extern "C" int tie_conv_qkv(const float* u, int row, const float* w, int taps, const float* state,
                            const int* state_slots, const int* seq_of_row, const int* query_start, int T, int nq,
                            int nk, int nv, const float* wq, const float* wk, float count_q, float count_k, float eps,
                            float* out, int out_row, hipStream_t stream) {
  const int C = nq + nk + nv;
  if (T <= 0 || C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || row < C || out_row < C ||
      static_cast<size_t>(C) * 4 > 65536 || (taps > 1 && !state))
    return TIE_BAD_ARGUMENT;
  const int threads = C >= 4096 ? 512 : (C >= 1024 ? 256 : 128);
  conv_qkv_kernel<<<T, threads, static_cast<size_t>(C) * sizeof(float), stream>>>(
      u, row, w, taps, state, state_slots, seq_of_row, query_start, nq, nk, nv, wq, wk, count_q, count_k, eps, out,
      out_row);
  return tie_launch_status();
}

// ---------------------------------------------------------------- the state of a short convolution after a step
// new[i] = input of row end - (taps - 1) + i: a row of this step, or what the old state held for it.
__global__ void conv_state_update_kernel(const float* __restrict__ u, int row, int taps, float* __restrict__ state,
                                         const int* __restrict__ state_slots, const int* __restrict__ query_start,
                                         int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = blockIdx.y;
  const int start = query_start[s], end = query_start[s + 1];
  const int hist = taps - 1;
  float* st = state + static_cast<size_t>(state_slots[s]) * hist * C;
  float keep[CONV_MAX_TAPS];
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
    if (i >= hist) break;
    const int src = end - hist + i;
    keep[i] = src >= start ? u[static_cast<size_t>(src) * row + c]
                           : st[static_cast<size_t>(src - start + hist) * C + c];
  }
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
    if (i >= hist) break;
    st[static_cast<size_t>(i) * C + c] = keep[i];
  }
}

extern "C" int tie_conv_state_update(const float* u, int row, int taps, float* state, const int* state_slots,
                                     const int* query_start, int num_seqs, int C, hipStream_t stream) {
  if (num_seqs <= 0 || C <= 0 || taps < 1 || taps > CONV_MAX_TAPS || row < C) return TIE_BAD_ARGUMENT;
  if (taps == 1) return TIE_OK;
  conv_state_update_kernel<<<dim3((C + 255) / 256, num_seqs), 256, 0, stream>>>(u, row, taps, state, state_slots,
                                                                                query_start, C);
  return tie_launch_status();
}

// ---------------------------------------------------------------- what the delta rule takes of a token
// Row t of `u`: [q (G d) | k (G d) | v (H e) | b (H)], the first C = 2 G d + H e columns convolved, then silu.
// Row t of `a`: the decay's argument (H d), `a_row` apart. out row: [q^ | k^ | v | beta (H) | g (H d)]:
//   q^, k^ unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q^ also times d^(-1/2); beta = sigmoid(b);
//   g = exp(-exp(A_log[head]) * softplus(a + dt_bias)).
__global__ void delta_prepare_kernel(const float* __restrict__ u, int row, const float* __restrict__ w, int taps,
                                     const float* __restrict__ state, const int* __restrict__ state_slots,
                                     const int* __restrict__ seq_of_row, const int* __restrict__ query_start,
                                     const float* __restrict__ a, int a_row, const float* __restrict__ A_log,
                                     const float* __restrict__ dt_bias, int G, int H, int d, int e,
                                     float* __restrict__ out, int out_row) {
  extern __shared__ float vals[];
  const int t = blockIdx.x;
  const int s = seq_of_row[t];
  const int start = query_start[s];
  const int C = 2 * G * d + H * e;
  const float* hist = state + static_cast<size_t>(state_slots[s]) * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const float y = taps > 1 ? conv_at(u, row, w, hist, taps, C, t, start, c)
                             : w[c] * u[static_cast<size_t>(t) * row + c];
    vals[c] = silu_f(y);
  }
  __syncthreads();
  float* o = out + static_cast<size_t>(t) * out_row;
  const int lane = threadIdx.x & (TIE_WAVE - 1), wave = threadIdx.x / TIE_WAVE, waves = blockDim.x / TIE_WAVE;
  const float q_scale = 1.0f / sqrtf(static_cast<float>(d));
  for (int head = wave; head < 2 * G; head += waves) {      // q heads, then k heads
    const float* x = vals + head * d;
    float ss = 0.f;
    for (int i = lane; i < d; i += TIE_WAVE) ss = fmaf(x[i], x[i], ss);
    const float inv = 1.0f / sqrtf(wave_sum(ss) + 1e-6f);
    const float f = head < G ? inv * q_scale : inv;
    for (int i = lane; i < d; i += TIE_WAVE) o[head * d + i] = x[i] * f;
  }
  for (int c = 2 * G * d + threadIdx.x; c < C; c += blockDim.x) o[c] = vals[c];
  const float* b = u + static_cast<size_t>(t) * row + C;
  for (int h = threadIdx.x; h < H; h += blockDim.x) o[C + h] = sigmoid_f(b[h]);
  const float* ar = a + static_cast<size_t>(t) * a_row;
  for (int c = threadIdx.x; c < H * d; c += blockDim.x)
    o[C + H + c] = expf(-expf(A_log[c / d]) * softplus_f(ar[c] + dt_bias[c]));
}

extern "C" int tie_delta_prepare(const float* u, int row, const float* w, int taps, const float* state,
                                 const int* state_slots, const int* seq_of_row, const int* query_start,
                                 const float* a, int a_row, const float* A_log, const float* dt_bias, int T, int G,
                                 int H, int d, int e, float* out, int out_row, hipStream_t stream) {
  const int C = 2 * G * d + H * e;
  if (T <= 0 || G <= 0 || H <= 0 || d <= 0 || e <= 0 || taps < 1 || taps > CONV_MAX_TAPS || row < C + H ||
      out_row < C + H + H * d || a_row < H * d || static_cast<size_t>(C) * 4 > 65536 || (taps > 1 && !state))
    return TIE_BAD_ARGUMENT;
  const int threads = C >= 2048 ? 512 : 256;
  delta_prepare_kernel<<<T, threads, static_cast<size_t>(C) * sizeof(float), stream>>>(
      u, row, w, taps, state, state_slots, seq_of_row, query_start, a, a_row, A_log, dt_bias, G, H, d, e, out,
      out_row);
  return tie_launch_status();
}

// ---------------------------------------------------------------- the recurrence
// A workgroup of four waves owns 64 value columns of one (sequence, value head). A lane is a column; wave p holds
// rows [p R, (p + 1) R) of that column in registers (R = key rows a wave: a quarter of key_dim rounded up to 8,
// 16, 32 or 64; rows beyond key_dim stay zero). The token's k, q and g lie in LDS, staged DELTA_TOKENS tokens at
// a time (the next ones are on their way meanwhile); every lane reads the same word of them, which LDS hands to
// a whole wave at once. The two sums over key rows (S^T k, S^T q) meet through LDS.
#define DELTA_TOKENS 4
#define DELTA_WAVES 4

template <int R>
__global__ __launch_bounds__(DELTA_WAVES* TIE_WAVE) void gated_delta_scan_kernel(
    const float* __restrict__ tok, int row, float* __restrict__ out, int out_row, float* __restrict__ state,
    const int* __restrict__ query_start, const int* __restrict__ state_slots, int G, int H, int d, int e) {
  constexpr int DP = R * DELTA_WAVES;                 // padded key rows
  __shared__ float kqg[DELTA_TOKENS][3][DP];
  __shared__ float vb[DELTA_TOKENS][TIE_WAVE + 1];    // the 64 values of the columns, then beta
  __shared__ float part[2][DELTA_WAVES][TIE_WAVE];
  const int s = blockIdx.x / H, head = blockIdx.x % H;
  const int kv = head / (H / G);
  const int lane = threadIdx.x & (TIE_WAVE - 1), p = threadIdx.x / TIE_WAVE;
  const int col = blockIdx.y * TIE_WAVE + lane;
  const bool live = col < e;
  const int t0 = query_start[s], t1 = query_start[s + 1];
  if (t0 >= t1) return;
  float* sp = state + ((static_cast<size_t>(state_slots[s]) * H + head) * d) * e + col;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p * R + r;
    S[r] = (live && i < d) ? sp[static_cast<size_t>(i) * e] : 0.f;
  }
  // column offsets inside a token's row
  const int q_at = kv * d, k_at = G * d + kv * d, v_at = 2 * G * d + head * e, b_at = 2 * G * d + H * e + head,
            g_at = 2 * G * d + H * e + H + head * d;
  constexpr int PER = (DELTA_TOKENS * 3 * DP + DELTA_WAVES * TIE_WAVE - 1) / (DELTA_WAVES * TIE_WAVE);
  float stage[PER], stage_v = 0.f, stage_b = 0.f;

  auto fetch = [&](int tb) {     // the tokens tb .. tb + DELTA_TOKENS - 1 into registers
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = j * (DELTA_WAVES * TIE_WAVE) + threadIdx.x;
      const int tk = idx / (3 * DP), rest = idx % (3 * DP), which = rest / DP, i = rest % DP;
      float v = which == 2 ? 1.f : 0.f;            // padding rows: no key, no query, no decay
      if (tk < DELTA_TOKENS && tb + tk < t1 && i < d) {
        const float* r = tok + static_cast<size_t>(tb + tk) * row;
        v = r[(which == 0 ? k_at : (which == 1 ? q_at : g_at)) + i];
      }
      stage[j] = v;
    }
    // values and beta: thread (p, lane) takes token p (DELTA_TOKENS == DELTA_WAVES)
    stage_v = stage_b = 0.f;
    if (tb + p < t1) {
      const float* r = tok + static_cast<size_t>(tb + p) * row;
      stage_v = live ? r[v_at + col] : 0.f;
      stage_b = r[b_at];
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int idx = j * (DELTA_WAVES * TIE_WAVE) + threadIdx.x;
      if (idx < DELTA_TOKENS * 3 * DP) (&kqg[0][0][0])[idx] = stage[j];
    }
    vb[p][lane] = stage_v;
    if (lane == 0) vb[p][TIE_WAVE] = stage_b;
  };

  fetch(t0);
  for (int tb = t0; tb < t1; tb += DELTA_TOKENS) {
    __syncthreads();          // everyone is done with the tokens staged before
    put();
    __syncthreads();
    if (tb + DELTA_TOKENS < t1) fetch(tb + DELTA_TOKENS);
    const int count = min(DELTA_TOKENS, t1 - tb);
    for (int j = 0; j < count; ++j) {
      const float* kk = &kqg[j][0][p * R];
      const float* qq = &kqg[j][1][p * R];
      const float* gg = &kqg[j][2][p * R];
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] *= gg[r];
        dot = fmaf(S[r], kk[r], dot);
      }
      part[0][p][lane] = dot;
      __syncthreads();
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < DELTA_WAVES; ++w) total += part[0][w][lane];
      const float u = vb[j][TIE_WAVE] * (vb[j][lane] - total);
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] = fmaf(kk[r], u, S[r]);
        o = fmaf(S[r], qq[r], o);
      }
      part[1][p][lane] = o;
      __syncthreads();
      if (p == 0 && live) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < DELTA_WAVES; ++w) sum += part[1][w][lane];
        out[static_cast<size_t>(tb + j) * out_row + head * e + col] = sum;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p * R + r;
    if (live && i < d) sp[static_cast<size_t>(i) * e] = S[r];
  }
}

// tok: rows of delta_prepare; out: float32 [T][>= H e]; state: [slots][H][d][e].
extern "C" int tie_gated_delta_scan(const float* tok, int row, float* out, int out_row, float* state,
                                    const int* query_start, const int* state_slots, int num_seqs, int G, int H, int d,
                                    int e, hipStream_t stream) {
  if (num_seqs <= 0 || G <= 0 || H <= 0 || H % G || d <= 0 || d > 256 || e <= 0 || out_row < H * e ||
      row < 2 * G * d + H * e + H + H * d)
    return TIE_BAD_ARGUMENT;
  const dim3 grid(num_seqs * H, (e + TIE_WAVE - 1) / TIE_WAVE);
  const int threads = DELTA_WAVES * TIE_WAVE;
#define SCAN(R)                                                                                                  \
  gated_delta_scan_kernel<R><<<grid, threads, 0, stream>>>(tok, row, out, out_row, state, query_start, state_slots, \
                                                           G, H, d, e)
  if (d <= 32) SCAN(8);
  else if (d <= 64) SCAN(16);
  else if (d <= 128) SCAN(32);
  else SCAN(64);
#undef SCAN
  return tie_launch_status();
}

// ---------------------------------------------------------------- the norm of the heads' outputs, gated
// out = o / rms(o over each group of `group` columns) * w[column in group] * sigmoid(gate), a wave a group.
template <typename TO>
__global__ void grouped_gated_rms_norm_kernel(const float* __restrict__ o, int o_row, const float* __restrict__ w,
                                              float eps, const float* __restrict__ gate, int gate_row,
                                              TO* __restrict__ out, int groups, int group) {
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int g = blockIdx.y * (blockDim.x / TIE_WAVE) + threadIdx.x / TIE_WAVE;
  if (g >= groups) return;
  const size_t t = blockIdx.x;
  const float* r = o + t * o_row + static_cast<size_t>(g) * group;
  const float* gt = gate + t * gate_row + static_cast<size_t>(g) * group;
  float ss = 0.f;
  for (int c = lane; c < group; c += TIE_WAVE) ss = fmaf(r[c], r[c], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(group) + eps);
  TO* d = out + (t * groups + g) * group;
  for (int c = lane; c < group; c += TIE_WAVE) store_from_float(d + c, (r[c] * inv) * w[c] * sigmoid_f(gt[c]));
}

extern "C" int tie_grouped_gated_rms_norm(const float* o, int o_row, const float* w, float eps, const float* gate,
                                          int gate_row, void* out, int out_dtype, int T, int groups, int group,
                                          hipStream_t stream) {
  if (T <= 0 || groups <= 0 || group <= 0 || o_row < groups * group || gate_row < groups * group)
    return TIE_BAD_ARGUMENT;
  const int waves = groups >= 4 ? 4 : groups;
  const dim3 grid(T, (groups + waves - 1) / waves);
  if (out_dtype == TIE_F32)
    grouped_gated_rms_norm_kernel<float><<<grid, waves * TIE_WAVE, 0, stream>>>(o, o_row, w, eps, gate, gate_row,
                                                                                static_cast<float*>(out), groups, group);
  else if (out_dtype == TIE_BF16)
    grouped_gated_rms_norm_kernel<bf16_t><<<grid, waves * TIE_WAVE, 0, stream>>>(
        o, o_row, w, eps, gate, gate_row, static_cast<bf16_t*>(out), groups, group);
  else
    return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}
