// Latent attention: what is cached of a token is one small latent vector c (kv_rank values, RMS-normed) and one
// rotated key part (rot values) shared by all heads. Head h's key is [W_uk[h] c | rotated part] and its value
// W_uv[h] c, so with the query's unrotated part taken through W_uk[h]^T first,
//     score = (W_uk[h]^T q_unrotated) . c + q_rotated . k_rotated ,
// attention runs over ONE key/value head of size kv_rank + rot whose values are the latents themselves, and
// W_uv[h] is applied to the attention's output. The kernels here make the cache rows and the rotated query parts
// (`latent_prepare`) and multiply every head by a matrix of its own (`head_linear`).
#include "common.h"

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---------------------------------------------------------------- cache rows and rotated query parts
// Row t of `proj` (float32, rows `row` apart): [q: H x (d + r) | c_raw (kr) | k_rot_raw (r) | ...]; where the queries
// come from a product of their own (queries made from a normed latent), `lat` (rows `lat_row` apart) holds
// [c_raw (kr) | k_rot_raw (r) | ...] instead and `proj` only the queries.
//   c = c_raw / rms(c_raw) * w_c                         -> key cache [c | rot(k_rot_raw) | 0 ..] (D columns) and
//                                                           value cache [c | 0 ..], transposed inside the page
//   q_unrot[t][h] (d values)                             -> qn (activation type), [T][H d]
//   rot(q_rot[t][h])                                     -> qa[t][h][kr .. kr + r), zeros behind up to D
// rot turns the first `rdims` of the r values by the angles of the token's position, pairs (2i, 2i + 1) where
// `interleaved`, else (i, i + rdims / 2); angles: [T][rdims] float32, the cosines then the sines.
template <typename TA, typename TC>
__global__ void latent_prepare_kernel(const float* __restrict__ proj, int row, const float* __restrict__ lat,
                                      int lat_row, const float* __restrict__ w_c, float eps,
                                      const float* __restrict__ angles, int rdims, int interleaved,
                                      const int* __restrict__ slots, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                      int block_size, int write_kv, TA* __restrict__ qn, TA* __restrict__ qa, int H,
                                      int d, int r, int kr, int D) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const float* p = proj + t * row;
  const float* ang = angles + t * rdims;
  const int half = rdims / 2;
  // the rotated value at place i of a vector x of r values
  auto rotated = [&](const float* x, int i) -> float {
    if (i >= rdims) return x[i];
    int pair, partner;
    bool first;
    if (interleaved) { pair = i >> 1; first = (i & 1) == 0; partner = first ? i + 1 : i - 1; }
    else { first = i < half; pair = first ? i : i - half; partner = first ? i + half : i - half; }
    const float c = ang[pair], s = ang[half + pair];
    return first ? x[i] * c - x[partner] * s : x[i] * c + x[partner] * s;
  };
  const int qw = d + r;
  // three workgroups a row, each with one part of the work: none waits for another's loads
  if (blockIdx.y == 0) {
    for (int i = threadIdx.x; i < H * d; i += blockDim.x) {
      const int h = i / d, j = i % d;
      store_from_float(qn + t * (static_cast<size_t>(H) * d) + i, p[h * qw + j]);
    }
    return;
  }
  if (blockIdx.y == 1) {
    for (int i = threadIdx.x; i < H * (D - kr); i += blockDim.x) {
      const int h = i / (D - kr), j = i % (D - kr);
      store_from_float(qa + (t * H + h) * D + kr + j, j < r ? rotated(p + h * qw + d, j) : 0.f);
    }
    return;
  }
  if (!write_kv) return;
  const float* c_raw = lat != nullptr ? lat + t * lat_row : p + H * qw;
  float ss = 0.f;
  for (int i = threadIdx.x; i < kr; i += blockDim.x) ss = fmaf(c_raw[i], c_raw[i], ss);
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(kr) + eps);
  const int slot = slots[t];
  const size_t page = slot / block_size, off = slot % block_size;
  TC* kd = k_cache + static_cast<size_t>(slot) * D;
  TC* vd = v_cache + page * D * block_size + off;
  for (int i = threadIdx.x; i < D; i += blockDim.x) {
    float kv = 0.f, vv = 0.f;
    if (i < kr) kv = vv = (c_raw[i] * inv) * w_c[i];
    else if (i < kr + r) kv = rotated(c_raw + kr, i - kr);
    store_from_float(kd + i, kv);
    store_from_float(vd + static_cast<size_t>(i) * block_size, vv);
  }
}

extern "C" int tie_latent_prepare(const float* proj, int row, const float* lat, int lat_row, const float* w_c,
                                  float eps, const float* angles,
                                  int rdims, int interleaved, const int* slots, void* k_cache, void* v_cache,
                                  int cache_dtype, int block_size, int write_kv, void* qn, void* qa, int act_dtype,
                                  int T, int H, int d, int r, int kr, int D, hipStream_t stream) {
  if (T <= 0 || H <= 0 || d <= 0 || r < 0 || kr <= 0 || D < kr + r || rdims < 0 || rdims > r || rdims % 2 ||
      row < H * (d + r) + (lat ? 0 : kr + r) || (lat && lat_row < kr + r) || block_size <= 0 || (rdims > 0 && !angles))
    return TIE_BAD_ARGUMENT;
  if (write_kv && (!slots || !k_cache || !v_cache)) return TIE_BAD_ARGUMENT;
  const int threads = 256;
#define LP(TA, TC)                                                                                                   \
  latent_prepare_kernel<TA, TC><<<dim3(T, 3), threads, 0, stream>>>(proj, row, lat, lat_row, w_c, eps, angles, rdims, interleaved, slots,   \
                                                           static_cast<TC*>(k_cache), static_cast<TC*>(v_cache),      \
                                                           block_size, write_kv, static_cast<TA*>(qn),                \
                                                           static_cast<TA*>(qa), H, d, r, kr, D)
  if (act_dtype == TIE_F32 && cache_dtype == TIE_F32) LP(float, float);
  else if (act_dtype == TIE_F32 && cache_dtype == TIE_BF16) LP(float, bf16_t);
  else if (act_dtype == TIE_F32 && cache_dtype == TIE_F16) LP(float, f16_t);
  else if (act_dtype == TIE_BF16 && cache_dtype == TIE_BF16) LP(bf16_t, bf16_t);
  else return TIE_BAD_ARGUMENT;
#undef LP
  return tie_launch_status();
}

// ---------------------------------------------------------------- an RMS norm over the first columns of wider rows
// out[t][i] = x[t][i] / sqrt(mean_i(x[t][i]^2) + eps) * w[i] for i < n, x rows `x_row` apart (float32), out dense.
template <typename TO>
__global__ void rms_norm_columns_kernel(const float* __restrict__ x, int x_row, const float* __restrict__ w, float eps,
                                        TO* __restrict__ out, int n) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const float* p = x + t * x_row;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(p[i], p[i], ss);
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) store_from_float(out + t * n + i, (p[i] * inv) * w[i]);
}

extern "C" int tie_rms_norm_columns(const float* x, int x_row, const float* w, float eps, void* out, int out_dtype,
                                    int T, int n, hipStream_t stream) {
  if (T <= 0 || n <= 0 || x_row < n) return TIE_BAD_ARGUMENT;
  const int threads = n >= 1024 ? 1024 : (n >= 256 ? 256 : 64);
  if (out_dtype == TIE_F32)
    rms_norm_columns_kernel<float><<<T, threads, 0, stream>>>(x, x_row, w, eps, static_cast<float*>(out), n);
  else if (out_dtype == TIE_BF16)
    rms_norm_columns_kernel<bf16_t><<<T, threads, 0, stream>>>(x, x_row, w, eps, static_cast<bf16_t*>(out), n);
  else return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}

// ---------------------------------------------------------------- a matrix of its own for every head
// out[t][h][n] = sum_k x[t][h][k] * w[h][n][k]   (n < N, k < K; float32 sums), optionally times sigmoid(gate[t][h][n]).
// x rows `x_row` apart with heads `x_head` apart, out likewise; w is [H][N][K] row-major. A workgroup of 256
// threads takes a tile of 64 rows x 64 columns of one head through LDS in steps of 16 along K; a thread 4 x 4.
#define HL_TILE 64
#define HL_K 16

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void head_linear_kernel(const TX* __restrict__ x, int x_row, int x_head,
                                                          const TW* __restrict__ w, TO* __restrict__ out, int out_row,
                                                          int out_head, const float* __restrict__ gate, int gate_row,
                                                          int gate_head, int T, int N, int K) {
  __shared__ float xs[HL_K][HL_TILE + 4];
  __shared__ float ws[HL_K][HL_TILE + 4];
  const int h = blockIdx.z;
  const int t0 = blockIdx.x * HL_TILE, n0 = blockIdx.y * HL_TILE;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;     // columns tx * 4 .., rows ty * 4 ..
  float acc[4][4] = {};
  const TW* wh = w + static_cast<size_t>(h) * N * K;
  for (int k0 = 0; k0 < K; k0 += HL_K) {
    for (int i = threadIdx.x; i < HL_TILE * HL_K; i += 256) {
      const int rr = i / HL_K, kk = i % HL_K;
      const int t = t0 + rr, n = n0 + rr, k = k0 + kk;
      xs[kk][rr] = (t < T && k < K) ? load_as_float(x + static_cast<size_t>(t) * x_row + h * x_head + k) : 0.f;
      ws[kk][rr] = (n < N && k < K) ? load_as_float(wh + static_cast<size_t>(n) * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HL_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = xs[kk][ty * 4 + i]; b[i] = ws[kk][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty * 4 + i;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (gate) v *= sigmoid_f(gate[static_cast<size_t>(t) * gate_row + h * gate_head + n]);
      store_from_float(out + static_cast<size_t>(t) * out_row + h * out_head + n, v);
    }
  }
}

// The same product on the matrix cores, for bfloat16 x and w whose rows of K start at multiples of 8 elements. A
// wave owns 16 rows x (NTILES x 16) columns of one head and reads its operands from memory in the very layout the
// 16x16x32 instruction takes them (eight consecutive k a lane), KSTEPS x 32 of K at a time, so those loads of a wave
// are under way before its first product. A lane ends with four consecutive columns of one row a tile, stored as one
// word where the sizes allow. Four waves a workgroup: side by side along the rows (ALONG_T, many
// rows) or along the columns (few rows: more waves share the heads' matrices). Float32 sums.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hl_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float hl_floatx4_t;
typedef uint32_t hl_u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ hl_bf16x8_t hl_frag(hl_u32x4_t v) { return *reinterpret_cast<const hl_bf16x8_t*>(&v); }

template <typename TO, int NTILES, bool ALONG_T>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(const bf16_t* __restrict__ x, int x_row, int x_head,
                                                               const bf16_t* __restrict__ w, TO* __restrict__ out,
                                                               int out_row, int out_head,
                                                               const float* __restrict__ gate, int gate_row,
                                                               int gate_head, int T, int N, int K, int whole) {
  const int h = blockIdx.z;
  const int wave = threadIdx.x / TIE_WAVE, lane = threadIdx.x % TIE_WAVE;
  const int t0 = (ALONG_T ? blockIdx.x * 4 + wave : blockIdx.x) * 16;
  const int n0 = (ALONG_T ? blockIdx.y : blockIdx.y * 4 + wave) * (NTILES * 16);
  if (t0 >= T || n0 >= N) return;                      // the whole wave; there is no barrier below
  const int r = lane % 16, kb = lane / 16;             // row of a fragment, block of 8 along k
  const bf16_t* xr = x + static_cast<size_t>(min(t0 + r, T - 1)) * x_row + h * x_head + kb * 8;
  const bf16_t* wr[NTILES];
#pragma unroll
  for (int i = 0; i < NTILES; ++i)
    wr[i] = w + (static_cast<size_t>(h) * N + min(n0 + i * 16 + r, N - 1)) * K + kb * 8;
  hl_floatx4_t acc[NTILES];
#pragma unroll
  for (int i = 0; i < NTILES; ++i) acc[i] = hl_floatx4_t{0.f, 0.f, 0.f, 0.f};
  const hl_u32x4_t zero = {0u, 0u, 0u, 0u};
  constexpr int KSTEPS = NTILES == 1 ? 8 : 4;
  for (int k0 = 0; k0 < K; k0 += KSTEPS * 32) {
    hl_u32x4_t xf[KSTEPS], wf[NTILES][KSTEPS];
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      if (k0 + st * 32 >= K) continue;
      const bool in = k0 + st * 32 + kb * 8 < K;
      xf[st] = in ? *reinterpret_cast<const hl_u32x4_t*>(xr + k0 + st * 32) : zero;
#pragma unroll
      for (int i = 0; i < NTILES; ++i)
        wf[i][st] = in ? *reinterpret_cast<const hl_u32x4_t*>(wr[i] + k0 + st * 32) : zero;
    }
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
      if (k0 + st * 32 >= K) continue;
#pragma unroll
      for (int i = 0; i < NTILES; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hl_frag(wf[i][st]), hl_frag(xf[st]), acc[i], 0, 0, 0);
    }
  }
  // a lane holds row t0 + lane % 16 and, of every tile, the four columns from (lane / 16) * 4 on
  const int t = t0 + r;
  if (t >= T) return;
#pragma unroll
  for (int i = 0; i < NTILES; ++i) {
    const int n = n0 + i * 16 + kb * 4;
    if (n >= N) continue;
    TO* o = out + static_cast<size_t>(t) * out_row + h * out_head + n;
    const float* g = gate ? gate + static_cast<size_t>(t) * gate_row + h * gate_head + n : nullptr;
    if (whole) {           // n + 3 < N, and four columns are one aligned word of out (and of gate)
      float y[4] = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
      if (g) {
        const float4 g4 = *reinterpret_cast<const float4*>(g);
        y[0] *= sigmoid_f(g4.x), y[1] *= sigmoid_f(g4.y), y[2] *= sigmoid_f(g4.z), y[3] *= sigmoid_f(g4.w);
      }
      if constexpr (sizeof(TO) == 2) {
        uint2 packed;
        packed.x = static_cast<uint32_t>(float_to_bf16(y[0])) | (static_cast<uint32_t>(float_to_bf16(y[1])) << 16);
        packed.y = static_cast<uint32_t>(float_to_bf16(y[2])) | (static_cast<uint32_t>(float_to_bf16(y[3])) << 16);
        *reinterpret_cast<uint2*>(o) = packed;
      } else {
        *reinterpret_cast<float4*>(o) = make_float4(y[0], y[1], y[2], y[3]);
      }
      continue;
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (n + v >= N) continue;
      float y = acc[i][v];
      if (g) y *= sigmoid_f(g[v]);
      store_from_float(o + v, y);
    }
  }
}

#define HL_FEW_ROWS 64     // up to here the four waves of a workgroup lie along the columns

template <typename TO>
static void launch_head_linear_mfma(const bf16_t* x, int x_row, int x_head, const bf16_t* w, TO* out, int out_row,
                                    int out_head, const float* gate, int gate_row, int gate_head, int T, int H, int N,
                                    int K, hipStream_t stream) {
  // four columns a store (and a gate load): sizes in steps of four from aligned addresses
  const int whole = N % 4 == 0 && out_row % 4 == 0 && out_head % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(out) % (4 * sizeof(TO)) == 0 &&
                    (!gate || (gate_row % 4 == 0 && gate_head % 4 == 0 && reinterpret_cast<uintptr_t>(gate) % 16 == 0));
  if (T <= HL_FEW_ROWS) {
    const dim3 grid((T + 15) / 16, (N + 63) / 64, H);
    head_linear_mfma_kernel<TO, 1, false><<<grid, 256, 0, stream>>>(x, x_row, x_head, w, out, out_row, out_head, gate,
                                                                    gate_row, gate_head, T, N, K, whole);
  } else {
    const dim3 grid((T + 63) / 64, (N + 63) / 64, H);
    head_linear_mfma_kernel<TO, 4, true><<<grid, 256, 0, stream>>>(x, x_row, x_head, w, out, out_row, out_head, gate,
                                                                   gate_row, gate_head, T, N, K, whole);
  }
}

extern "C" int tie_head_linear(const void* x, int x_dtype, int x_row, int x_head, const void* w, int w_dtype, void* out,
                               int out_dtype, int out_row, int out_head, const float* gate, int gate_row,
                               int gate_head, int T, int H, int N, int K, hipStream_t stream) {
  if (T <= 0 || H <= 0 || N <= 0 || K <= 0 || H > 65535 || (T + 15) / 16 > 65535 * 4) return TIE_BAD_ARGUMENT;
  if (x_dtype == TIE_BF16 && w_dtype == TIE_BF16 && (out_dtype == TIE_BF16 || out_dtype == TIE_F32) && K % 8 == 0 &&
      x_row % 8 == 0 && x_head % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    if (out_dtype == TIE_BF16)
      launch_head_linear_mfma(static_cast<const bf16_t*>(x), x_row, x_head, static_cast<const bf16_t*>(w),
                              static_cast<bf16_t*>(out), out_row, out_head, gate, gate_row, gate_head, T, H, N, K, stream);
    else
      launch_head_linear_mfma(static_cast<const bf16_t*>(x), x_row, x_head, static_cast<const bf16_t*>(w),
                              static_cast<float*>(out), out_row, out_head, gate, gate_row, gate_head, T, H, N, K, stream);
    return tie_launch_status();
  }
  const dim3 grid((T + HL_TILE - 1) / HL_TILE, (N + HL_TILE - 1) / HL_TILE, H);
#define HL(TX, TW, TO)                                                                                              \
  head_linear_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>(static_cast<const TX*>(x), x_row, x_head,               \
                                                           static_cast<const TW*>(w), static_cast<TO*>(out), out_row, \
                                                           out_head, gate, gate_row, gate_head, T, N, K)
  if (x_dtype == TIE_F32 && w_dtype == TIE_F32 && out_dtype == TIE_F32) HL(float, float, float);
  else if (x_dtype == TIE_BF16 && w_dtype == TIE_BF16 && out_dtype == TIE_BF16) HL(bf16_t, bf16_t, bf16_t);
  else if (x_dtype == TIE_BF16 && w_dtype == TIE_BF16 && out_dtype == TIE_F32) HL(bf16_t, bf16_t, float);
  else if (x_dtype == TIE_F32 && w_dtype == TIE_BF16 && out_dtype == TIE_F32) HL(float, bf16_t, float);
  else return TIE_BAD_ARGUMENT;
#undef HL
  return tie_launch_status();
}
