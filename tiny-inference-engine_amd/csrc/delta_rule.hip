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
  // three workgroups a row: q, k and v each on their own (a norm runs over one of them)
  const int lo = blockIdx.y == 0 ? 0 : (blockIdx.y == 1 ? nq : nq + nk);
  const int hi = blockIdx.y == 0 ? nq : (blockIdx.y == 1 ? nq + nk : C);
  float sq = 0.f, sk = 0.f;
  for (int c = lo + threadIdx.x; c < hi; c += blockDim.x) {
    const float y = taps > 1 ? conv_at(u, row, w, hist, taps, C, t, start, c)
                             : w[c] * u[static_cast<size_t>(t) * row + c];
    vals[c] = y;
    if (c < nq) sq = fmaf(y, y, sq);
    else if (c < nq + nk) sk = fmaf(y, y, sk);
  }
  float iq = 1.f, ik = 1.f;
  if (wq && blockIdx.y == 0) iq = 1.0f / sqrtf(block_sum(sq, scratch) / count_q + eps);
  if (wk && blockIdx.y == 1) ik = 1.0f / sqrtf(block_sum(sk, scratch) / count_k + eps);
  __syncthreads();
  float* o = out + static_cast<size_t>(t) * out_row;
  for (int c = lo + threadIdx.x; c < hi; c += blockDim.x) {
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
  // few channels a thread: every one waits for its loads, and a decode step brings few rows
  const int threads = C >= 2048 ? 1024 : (C >= 1024 ? 512 : (C >= 512 ? 256 : 128));
  conv_qkv_kernel<<<dim3(T, 3), threads, static_cast<size_t>(C) * sizeof(float), stream>>>(
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
// Row t of `a`: the decay's argument (H d), `a_row` apart. out row: [q^ | k^ | v | g (H d) | beta (H)]:
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
  float* o = out + static_cast<size_t>(t) * out_row;
  // three workgroups a row: q and k with their unit norms, v, and beta with the decays
  if (blockIdx.y == 2) {
    const float* b = u + static_cast<size_t>(t) * row + C;
    for (int h = threadIdx.x; h < H; h += blockDim.x) o[C + H * d + h] = sigmoid_f(b[h]);
    const float* ar = a + static_cast<size_t>(t) * a_row;
    for (int c = threadIdx.x; c < H * d; c += blockDim.x)
      o[C + c] = expf(-expf(A_log[c / d]) * softplus_f(ar[c] + dt_bias[c]));
    return;
  }
  const int lo = blockIdx.y == 0 ? 0 : 2 * G * d, hi = blockIdx.y == 0 ? 2 * G * d : C;
  for (int c = lo + threadIdx.x; c < hi; c += blockDim.x) {
    const float y = taps > 1 ? conv_at(u, row, w, hist, taps, C, t, start, c)
                             : w[c] * u[static_cast<size_t>(t) * row + c];
    if (blockIdx.y == 0) vals[c] = silu_f(y);
    else o[c] = silu_f(y);
  }
  if (blockIdx.y == 1) return;
  __syncthreads();
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
}

extern "C" int tie_delta_prepare(const float* u, int row, const float* w, int taps, const float* state,
                                 const int* state_slots, const int* seq_of_row, const int* query_start,
                                 const float* a, int a_row, const float* A_log, const float* dt_bias, int T, int G,
                                 int H, int d, int e, float* out, int out_row, hipStream_t stream) {
  const int C = 2 * G * d + H * e;
  if (T <= 0 || G <= 0 || H <= 0 || d <= 0 || e <= 0 || taps < 1 || taps > CONV_MAX_TAPS || row < C + H ||
      out_row < C + H + H * d || a_row < H * d || static_cast<size_t>(C) * 4 > 65536 || (taps > 1 && !state))
    return TIE_BAD_ARGUMENT;
  const int threads = C >= 2048 ? 1024 : (C >= 1024 ? 512 : 256);
  delta_prepare_kernel<<<dim3(T, 3), threads, static_cast<size_t>(C) * sizeof(float), stream>>>(
      u, row, w, taps, state, state_slots, seq_of_row, query_start, a, a_row, A_log, dt_bias, G, H, d, e, out,
      out_row);
  return tie_launch_status();
}

// ---------------------------------------------------------------- the recurrence
// A wave owns DELTA_COLS value columns of one (sequence, value head): lane l holds rows [p R, (p + 1) R) of column
// l / 8 in registers, p = l % 8 (R = key rows a lane: an eighth of key_dim rounded up to 4, 8, 16 or 32; rows
// beyond key_dim stay zero), so the two sums over key rows (S^T k, S^T q) meet inside eight neighbouring lanes,
// through three lane permutations each and without a barrier. The DELTA_WAVES waves of a workgroup take columns
// side by side and share the token's k, q and g in LDS, staged NT tokens at a time (the next ones are on their way
// from memory meanwhile, four words a load where the row's layout allows), every p's rows four words behind the
// last one's so that the eight addresses of one read fall into different banks; the lanes of one p read the same
// words. A token's words are in registers before the token before it is done.
#define DELTA_COLS 8
#define DELTA_PARTS 8
#define DELTA_WAVES 4
#define DELTA_THREADS (DELTA_WAVES * TIE_WAVE)

__device__ __forceinline__ float part_sum(float v) {     // over the DELTA_PARTS lanes of a column
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));
  return v;
}

// Where a head's columns lie inside a token's row, and where the sequence's tokens end.
struct DeltaRowPlan {
  int k_at, q_at, g_at, v_at, b_at, first_col, d, e, t1, row;
};

// k, q and g of the tokens tb .. tb + NT - 1 of the head (padded to DP rows) into registers, W words a load:
// entry (x * DELTA_THREADS + thread) * W of [token][k, q, g][row]. Every load is issued whether it counts or not
// (from an address that exists), so that none waits for a branch.
template <int DP, int NT, int W, int PER>
__device__ __forceinline__ void delta_fetch(const float* __restrict__ tok, const DeltaRowPlan pl, int tb,
                                            float (&stage)[PER][W]) {
  const float* first = tok + static_cast<size_t>(tb) * pl.row;
  const int left = pl.t1 - tb;                    // tokens from tb on, at least one
#pragma unroll
  for (int x = 0; x < PER; ++x) {
    const int idx = (x * DELTA_THREADS + static_cast<int>(threadIdx.x)) * W;
    const int tk = idx / (3 * DP), rest = idx % (3 * DP), which = rest / DP, i = rest % DP;
    const float* r = first + static_cast<size_t>(min(tk, left - 1)) * pl.row +
                     (which == 0 ? pl.k_at : (which == 1 ? pl.q_at : pl.g_at));
    const float pad = which == 2 ? 1.f : 0.f;      // padding rows: no key, no query, no decay
    if constexpr (W == 4) {                        // d is a multiple of 4: the four rows count together
      const float4 v = *reinterpret_cast<const float4*>(r + min(i, pl.d - 4));
      const bool in = tk < left && i < pl.d;
      stage[x][0] = in ? v.x : pad, stage[x][1] = in ? v.y : pad, stage[x][2] = in ? v.z : pad, stage[x][3] = in ? v.w : pad;
    } else {
      const float v = r[min(i, pl.d - 1)];
      stage[x][0] = (tk < left && i < pl.d) ? v : pad;
    }
  }
}

// The values of the wave's columns and beta of the same tokens: entry j * 64 + lane of [token][columns, beta].
template <int NT, int VB>
__device__ __forceinline__ void delta_fetch_values(const float* __restrict__ tok, const DeltaRowPlan pl, int tb,
                                                   int lane, float (&stage_vb)[VB]) {
  const float* first = tok + static_cast<size_t>(tb) * pl.row;
  const int left = pl.t1 - tb;
#pragma unroll
  for (int j = 0; j < VB; ++j) {
    const int idx = j * TIE_WAVE + lane;
    const int tk = idx / (DELTA_COLS + 1), x = idx % (DELTA_COLS + 1);
    const float* r = first + static_cast<size_t>(min(tk, left - 1)) * pl.row;
    const float v = r[x == DELTA_COLS ? pl.b_at : pl.v_at + min(pl.first_col + x, pl.e - 1)];
    stage_vb[j] = (tk < NT && tk < left && (x == DELTA_COLS || pl.first_col + x < pl.e)) ? v : 0.f;
  }
}

// One token through the lane's rows: S <- g S; u = beta (v - S^T k); S <- S + k u; returns S^T q.
template <int R>
__device__ __forceinline__ float delta_token(float (&S)[R], const float (&kk)[R], const float (&qq)[R],
                                             const float (&gg)[R], float v, float beta) {
  float dot0 = 0.f, dot1 = 0.f, dot2 = 0.f, dot3 = 0.f;
#pragma unroll
  for (int r = 0; r < R; r += 4) {
    S[r] *= gg[r];
    S[r + 1] *= gg[r + 1];
    S[r + 2] *= gg[r + 2];
    S[r + 3] *= gg[r + 3];
    dot0 = fmaf(S[r], kk[r], dot0);
    dot1 = fmaf(S[r + 1], kk[r + 1], dot1);
    dot2 = fmaf(S[r + 2], kk[r + 2], dot2);
    dot3 = fmaf(S[r + 3], kk[r + 3], dot3);
  }
  const float u = beta * (v - part_sum((dot0 + dot1) + (dot2 + dot3)));
  float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
  for (int r = 0; r < R; r += 4) {
    S[r] = fmaf(kk[r], u, S[r]);
    S[r + 1] = fmaf(kk[r + 1], u, S[r + 1]);
    S[r + 2] = fmaf(kk[r + 2], u, S[r + 2]);
    S[r + 3] = fmaf(kk[r + 3], u, S[r + 3]);
    o0 = fmaf(S[r], qq[r], o0);
    o1 = fmaf(S[r + 1], qq[r + 1], o1);
    o2 = fmaf(S[r + 2], qq[r + 2], o2);
    o3 = fmaf(S[r + 3], qq[r + 3], o3);
  }
  return part_sum((o0 + o1) + (o2 + o3));
}

// What a launch of the scan walks. Without `items` a workgroup's rows are a sequence's rows of the step and its
// state the sequence's slot. With `items` ([count][3]: sequence, first row, end row) they are one chunk's, and the
// state is entry `item` of `state`. A state has `columns` columns: e, or e + d where the columns from e on carry the
// chunk's transition (they start as the identity and take no values, so they end as the product of the tokens'
// transition matrices, which is what the state before the chunk is multiplied by).
struct DeltaScanMode {
  const int* items;
  int columns;
  int init;      // 0: the state is read; 1: it starts as zeros (and the identity from column e on)
  int store;     // the state is written back at the end
  int outputs;   // outputs are written
};

template <int R, int W>
__global__ __launch_bounds__(DELTA_THREADS) void gated_delta_scan_kernel(
    const float* __restrict__ tok, int row, float* __restrict__ out, int out_row, float* __restrict__ state,
    const int* __restrict__ query_start, const int* __restrict__ state_slots, int G, int H, int d, int e,
    DeltaScanMode mode) {
  constexpr int DP = R * DELTA_PARTS;                 // padded key rows
  constexpr int RP = R + 4;                           // words from one p's rows to the next one's in LDS
  constexpr int NT = 4 * DELTA_THREADS / DP;          // tokens staged at a time: 4 to 32
  constexpr int PER = NT * 3 * DP / (DELTA_THREADS * W);
  constexpr int VB = (NT * (DELTA_COLS + 1) + TIE_WAVE - 1) / TIE_WAVE;
  __shared__ __attribute__((aligned(16))) float kqg[NT * 3 * DELTA_PARTS * RP];   // [token][k, q, g][p][row]
  __shared__ float vbs[DELTA_WAVES][NT * (DELTA_COLS + 1)];     // a wave: [token][the values of its columns, beta]
  const int item = blockIdx.x / H, head = blockIdx.x % H;
  const int kv = head / (H / G);
  const int wave = threadIdx.x / TIE_WAVE, lane = threadIdx.x % TIE_WAVE;
  const int p = lane & (DELTA_PARTS - 1), c = lane / DELTA_PARTS;
  const int first_col = (blockIdx.y * DELTA_WAVES + wave) * DELTA_COLS;
  const int col = first_col + c;
  const int columns = mode.columns;
  const bool live = col < columns;
  int t0, t1, holder;
  if (mode.items) {
    t0 = mode.items[3 * item + 1], t1 = mode.items[3 * item + 2], holder = item;
  } else {
    t0 = query_start[item], t1 = query_start[item + 1], holder = state_slots[item];
  }
  if (t0 >= t1) return;                               // the whole workgroup
  float* sp = state + ((static_cast<size_t>(holder) * H + head) * d) * columns + col;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p * R + r;
    if (mode.init) S[r] = (live && col - e == i) ? 1.f : 0.f;
    else S[r] = (live && i < d) ? sp[static_cast<size_t>(i) * columns] : 0.f;
  }
  DeltaRowPlan pl;
  pl.q_at = kv * d;
  pl.k_at = G * d + kv * d;
  pl.v_at = 2 * G * d + head * e;
  pl.g_at = 2 * G * d + H * e + head * d;
  pl.b_at = 2 * G * d + H * e + H * d + head;
  pl.first_col = first_col;
  pl.d = d, pl.e = e, pl.t1 = t1, pl.row = row;
  float* vb = vbs[wave];
  const bool writes = mode.outputs && p == 0 && col < e;
  float stage[PER][W], stage_vb[VB];
  delta_fetch<DP, NT, W, PER>(tok, pl, t0, stage);
  delta_fetch_values<NT, VB>(tok, pl, t0, lane, stage_vb);
  float ka[R], qa[R], ga[R], kb[R], qb[R], gb[R];
  auto read = [&](int j, float (&kk)[R], float (&qq)[R], float (&gg)[R]) {     // token j of the staged ones
    const float* at = kqg + (j * 3 * DELTA_PARTS + p) * RP;
#pragma unroll
    for (int r = 0; r < R; r += 4) {
      const float4 k4 = *reinterpret_cast<const float4*>(at + r);
      const float4 q4 = *reinterpret_cast<const float4*>(at + DELTA_PARTS * RP + r);
      const float4 g4 = *reinterpret_cast<const float4*>(at + 2 * DELTA_PARTS * RP + r);
      kk[r] = k4.x, kk[r + 1] = k4.y, kk[r + 2] = k4.z, kk[r + 3] = k4.w;
      qq[r] = q4.x, qq[r + 1] = q4.y, qq[r + 2] = q4.z, qq[r + 3] = q4.w;
      gg[r] = g4.x, gg[r + 1] = g4.y, gg[r + 2] = g4.z, gg[r + 3] = g4.w;
    }
  };
  for (int tb = t0; tb < t1; tb += NT) {
    __syncthreads();          // every wave is done with the tokens staged before
#pragma unroll
    for (int x = 0; x < PER; ++x) {                  // [token][which][row] as fetched
      const int idx = (x * DELTA_THREADS + static_cast<int>(threadIdx.x)) * W;
      const int vec = idx / DP, i = idx % DP;
      float* to = kqg + (vec * DELTA_PARTS + i / R) * RP + i % R;
      if constexpr (W == 4) {
        *reinterpret_cast<float4*>(to) = make_float4(stage[x][0], stage[x][1], stage[x][2], stage[x][3]);
      } else {
        *to = stage[x][0];
      }
    }
#pragma unroll
    for (int j = 0; j < VB; ++j) {
      const int idx = j * TIE_WAVE + lane;
      if (idx < NT * (DELTA_COLS + 1)) vb[idx] = stage_vb[j];
    }
    __syncthreads();
    if (tb + NT < t1) {
      delta_fetch<DP, NT, W, PER>(tok, pl, tb + NT, stage);
      delta_fetch_values<NT, VB>(tok, pl, tb + NT, lane, stage_vb);
    }
    const int count = min(NT, t1 - tb);
    float* o = out + static_cast<size_t>(tb) * out_row + head * e + col;
    if constexpr (R > 16) {   // too many rows a lane for two tokens' words in registers
      for (int j = 0; j < count; ++j) {
        read(j, ka, qa, ga);
        const float sum = delta_token<R>(S, ka, qa, ga, vb[j * (DELTA_COLS + 1) + c], vb[j * (DELTA_COLS + 1) + DELTA_COLS]);
        if (writes) o[static_cast<size_t>(j) * out_row] = sum;
      }
      continue;
    }
    read(0, ka, qa, ga);
    for (int j = 0; j < count; j += 2) {
      if (j + 1 < count) read(j + 1, kb, qb, gb);
      const float first = delta_token<R>(S, ka, qa, ga, vb[j * (DELTA_COLS + 1) + c], vb[j * (DELTA_COLS + 1) + DELTA_COLS]);
      if (writes) o[static_cast<size_t>(j) * out_row] = first;
      if (j + 1 < count) {
        if (j + 2 < count) read(j + 2, ka, qa, ga);
        const float second = delta_token<R>(S, kb, qb, gb, vb[(j + 1) * (DELTA_COLS + 1) + c],
                                            vb[(j + 1) * (DELTA_COLS + 1) + DELTA_COLS]);
        if (writes) o[static_cast<size_t>(j + 1) * out_row] = second;
      }
    }
  }
  if (!mode.store) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p * R + r;
    if (live && i < d) sp[static_cast<size_t>(i) * columns] = S[r];
  }
}

// The chunks' states in order: `ends` [count][H][d][e + d] holds what every chunk makes of a zero state (columns
// below e) and its transition P (columns from e on). A workgroup owns COMBINE_COLS columns of a (sequence, head):
// it leaves every chunk the state before its first token (`starts` [count][H][d][e]) and the slot the state behind
// the last one, S <- P S + L chunk after chunk. A thread has a row (two where d > 128) and four columns; the state
// lies in LDS, and P passes through LDS `jt` columns at a time (rows jt + 1 words apart: the rows of a wave meet
// different banks), the next tile on its way into registers meanwhile.
#define COMBINE_COLS 8
#define COMBINE_THREADS 256
#define COMBINE_TILE 8192          // elements of P in LDS at a time
#define COMBINE_PER (COMBINE_TILE / COMBINE_THREADS)

__global__ __launch_bounds__(COMBINE_THREADS) void gated_delta_combine_kernel(
    const float* __restrict__ ends, float* __restrict__ starts, float* __restrict__ state,
    const int* __restrict__ first_chunk, const int* __restrict__ state_slots, int H, int d, int e, int jt) {
  extern __shared__ __attribute__((aligned(16))) float sl[];       // [2][d][COMBINE_COLS], then P's tile [d][jt + 1]
  const int s = blockIdx.x / H, head = blockIdx.x % H;
  const int c0 = first_chunk[s], c1 = first_chunk[s + 1];
  if (c0 >= c1) return;
  const int col0 = blockIdx.y * COMBINE_COLS;
  const int half = threadIdx.x & 1, col = col0 + half * 4;          // this thread's four columns
  const int row0 = threadIdx.x >> 1;                                // its rows: row0, row0 + 128
  float* slot = state + (static_cast<size_t>(state_slots[s]) * H + head) * d * e;
  float* cur = sl;
  float* nxt = sl + d * COMBINE_COLS;
  float* pl = sl + 2 * d * COMBINE_COLS;
  for (int i = row0; i < d; i += COMBINE_THREADS / 2)
#pragma unroll
    for (int x = 0; x < 4; ++x) cur[i * COMBINE_COLS + half * 4 + x] = col + x < e ? slot[static_cast<size_t>(i) * e + col + x] : 0.f;
  const int wide = e + d;
  const int tiles = (d + jt - 1) / jt;
  float ahead[COMBINE_PER];
  // element k * COMBINE_THREADS + thread of a tile is (row, column) = (i0 + k * rows_step, jj0) where jt divides the
  // threads; otherwise a division an element
  const bool regular = COMBINE_THREADS % jt == 0;
  const int i0 = threadIdx.x / jt, jj0 = threadIdx.x % jt, rows_step = COMBINE_THREADS / jt;
  auto fetch = [&](int c, int tile) {            // tile `tile` of chunk c's P into registers
    const float* P = ends + (static_cast<size_t>(c) * H + head) * d * wide + e + tile * jt;
    const int width = min(jt, d - tile * jt);
#pragma unroll
    for (int k = 0; k < COMBINE_PER; ++k) {
      int i = i0 + k * rows_step, jj = jj0;
      if (!regular) i = (k * COMBINE_THREADS + threadIdx.x) / jt, jj = (k * COMBINE_THREADS + threadIdx.x) % jt;
      ahead[k] = (i < d && jj < width) ? P[static_cast<size_t>(i) * wide + jj] : 0.f;
    }
  };
  fetch(c0, 0);
  float acc[2][4];
  for (int c = c0; c < c1; ++c) {
    const float* E = ends + (static_cast<size_t>(c) * H + head) * d * wide;
    float* st = starts + (static_cast<size_t>(c) * H + head) * d * e;
    for (int tile = 0; tile < tiles; ++tile) {
      __syncthreads();                             // the tile before is used up; `cur` is whole
#pragma unroll
      for (int k = 0; k < COMBINE_PER; ++k) {
        int i = i0 + k * rows_step, jj = jj0;
        if (!regular) i = (k * COMBINE_THREADS + threadIdx.x) / jt, jj = (k * COMBINE_THREADS + threadIdx.x) % jt;
        if (i < d) pl[i * (jt + 1) + jj] = ahead[k];
      }
      __syncthreads();
      if (tile + 1 < tiles) fetch(c, tile + 1);
      else if (c + 1 < c1) fetch(c + 1, 0);
      const int width = min(jt, d - tile * jt);
#pragma unroll
      for (int rr = 0; rr < 2; ++rr) {
        const int i = row0 + rr * (COMBINE_THREADS / 2);
        if (i >= d) continue;
        if (tile == 0) {
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            if (col + x < e) st[static_cast<size_t>(i) * e + col + x] = cur[i * COMBINE_COLS + half * 4 + x];
            acc[rr][x] = col + x < e ? E[static_cast<size_t>(i) * wide + col + x] : 0.f;
          }
        }
        const float* pi = pl + i * (jt + 1);
        const float* sj = cur + tile * jt * COMBINE_COLS + half * 4;
        for (int jj = 0; jj < width; ++jj) {
          const float pij = pi[jj];
          const float4 v = *reinterpret_cast<const float4*>(sj + jj * COMBINE_COLS);
          acc[rr][0] = fmaf(pij, v.x, acc[rr][0]);
          acc[rr][1] = fmaf(pij, v.y, acc[rr][1]);
          acc[rr][2] = fmaf(pij, v.z, acc[rr][2]);
          acc[rr][3] = fmaf(pij, v.w, acc[rr][3]);
        }
        if (tile + 1 == tiles) {
#pragma unroll
          for (int x = 0; x < 4; ++x) nxt[i * COMBINE_COLS + half * 4 + x] = acc[rr][x];
        }
      }
    }
    float* t = cur;
    cur = nxt;
    nxt = t;
  }
  __syncthreads();
  for (int i = row0; i < d; i += COMBINE_THREADS / 2)
#pragma unroll
    for (int x = 0; x < 4; ++x)
      if (col + x < e) slot[static_cast<size_t>(i) * e + col + x] = cur[i * COMBINE_COLS + half * 4 + x];
}

// tok: rows of delta_prepare; out: float32 [T][>= H e]; state: [slots][H][d][e].
static int launch_delta_scan(const float* tok, int row, float* out, int out_row, float* state, const int* query_start,
                             const int* state_slots, int num_items, int G, int H, int d, int e, DeltaScanMode mode,
                             hipStream_t stream) {
  constexpr int wg_cols = DELTA_WAVES * DELTA_COLS;
  const dim3 grid(num_items * H, (mode.columns + wg_cols - 1) / wg_cols);
  if (grid.y > 65535) return TIE_BAD_ARGUMENT;
  // four words a load where every head's k, q and g start at a multiple of four words of an aligned row
  const bool wide = d % 4 == 0 && (H * e) % 4 == 0 && row % 4 == 0 && reinterpret_cast<uintptr_t>(tok) % 16 == 0;
#define SCAN(R)                                                                                                    \
  do {                                                                                                             \
    if (wide)                                                                                                      \
      gated_delta_scan_kernel<R, 4><<<grid, DELTA_THREADS, 0, stream>>>(tok, row, out, out_row, state, query_start, \
                                                                        state_slots, G, H, d, e, mode);             \
    else                                                                                                           \
      gated_delta_scan_kernel<R, 1><<<grid, DELTA_THREADS, 0, stream>>>(tok, row, out, out_row, state, query_start, \
                                                                        state_slots, G, H, d, e, mode);             \
  } while (0)
  if (d <= 32) SCAN(4);
  else if (d <= 64) SCAN(8);
  else if (d <= 128) SCAN(16);
  else SCAN(32);
#undef SCAN
  return tie_launch_status();
}

extern "C" int tie_gated_delta_scan(const float* tok, int row, float* out, int out_row, float* state,
                                    const int* query_start, const int* state_slots, int num_seqs, int G, int H, int d,
                                    int e, hipStream_t stream) {
  if (num_seqs <= 0 || G <= 0 || H <= 0 || H % G || d <= 0 || d > 256 || e <= 0 || out_row < H * e ||
      row < 2 * G * d + H * e + H + H * d)
    return TIE_BAD_ARGUMENT;
  return launch_delta_scan(tok, row, out, out_row, state, query_start, state_slots, num_seqs, G, H, d, e,
                           DeltaScanMode{nullptr, e, 0, 1, 1}, stream);
}

// The same over chunks, in three launches: every chunk from a zero state with its transition beside it (`ends`
// [count][H][d][e + d]), the chunks' states combined in order (`starts` [count][H][d][e]; the slots receive the
// final states), every chunk again from its true start with outputs. items: [count][3] (sequence, first row, end
// row), in the order of the sequences' rows; first_chunk: [num_seqs + 1].
extern "C" int tie_gated_delta_scan_chunked(const float* tok, int row, float* out, int out_row, float* state,
                                            const int* state_slots, int num_seqs, const int* items,
                                            const int* first_chunk, int count, float* ends, float* starts, int G,
                                            int H, int d, int e, hipStream_t stream) {
  if (num_seqs <= 0 || count <= 0 || G <= 0 || H <= 0 || H % G || d <= 0 || d > 256 || e <= 0 || out_row < H * e ||
      row < 2 * G * d + H * e + H + H * d || !items || !first_chunk || !ends || !starts)
    return TIE_BAD_ARGUMENT;
  int rc = launch_delta_scan(tok, row, out, out_row, ends, nullptr, nullptr, count, G, H, d, e,
                             DeltaScanMode{items, e + d, 1, 1, 0}, stream);
  if (rc != TIE_OK) return rc;
  const dim3 grid(num_seqs * H, (e + COMBINE_COLS - 1) / COMBINE_COLS);
  if (grid.y > 65535) return TIE_BAD_ARGUMENT;
  int jt = COMBINE_TILE / d / 4 * 4;           // d <= 256: at least 32
  if (jt > d) jt = d;
  const size_t lds = (2 * static_cast<size_t>(d) * COMBINE_COLS + static_cast<size_t>(d) * (jt + 1)) * sizeof(float);
  gated_delta_combine_kernel<<<grid, COMBINE_THREADS, lds, stream>>>(ends, starts, state, first_chunk, state_slots, H,
                                                                     d, e, jt);
  rc = tie_launch_status();
  if (rc != TIE_OK) return rc;
  return launch_delta_scan(tok, row, out, out_row, starts, nullptr, nullptr, count, G, H, d, e,
                           DeltaScanMode{items, e, 0, 0, 1}, stream);
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
