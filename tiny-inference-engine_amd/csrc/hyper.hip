// Layer norm without a bias, and hyper-connections: several residual streams that every sub-layer reads as one
// weighted sum and updates all at once.
//
//   read:   u = sum_s in[s] x_s ;  h = norm(u) * w
//   write:  x_t <- sum_s mix[s][t] x_s + out[t] y      for every t, from the old streams
//
// One workgroup takes one row. A launch does, in this order and each only if asked for: the write of the sub-layer
// that just ended (y as rows, or as planes of partial sums that are added in plane order), the sum of the streams into the model's single residual row, and the read for the sub-layer that comes
// next with its norm. Streams that do not exist yet (the first sub-layer of a step) are all equal to the row of
// `x`. Everything is float32 but the normed rows, which take the activation type.
#include "common.h"

#define HYPER_MAX_STREAMS 8

// ------------------------------------------------------------------ layer norm
// out = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w, the variance from the deviations (two passes over a row
// that lies in LDS), float32 statistics. `rows` (or null) picks the rows of x that are normed.
template <typename TX, typename TO>
__global__ void layer_norm_kernel(const TX* __restrict__ x, const float* __restrict__ w, float eps, TO* __restrict__ out,
                                  const int* __restrict__ rows, int n) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const size_t src = rows ? static_cast<size_t>(rows[blockIdx.x]) : blockIdx.x;
  const TX* r = x + src * n;
  float sum = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = load_as_float(r + c);
    row[c] = v;
    sum += v;
  }
  const float mean = block_sum(sum, scratch) / static_cast<float>(n);
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float d = row[c] - mean;
    ss = fmaf(d, d, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + eps);
  TO* o = out + static_cast<size_t>(blockIdx.x) * n;
  for (int c = threadIdx.x; c < n; c += blockDim.x) store_from_float(o + c, ((row[c] - mean) * inv) * w[c]);
}

static int row_threads(int n) { return n >= 4096 ? 512 : (n >= 1024 ? 256 : (n >= 256 ? 128 : 64)); }

extern "C" int tie_layer_norm(const void* x, int x_dtype, const float* w, float eps, void* out, int out_dtype,
                              const int* rows, int count, int n, hipStream_t stream) {
  if (count <= 0 || n <= 0 || static_cast<size_t>(n) * 4 > 65536) return TIE_BAD_ARGUMENT;
  const int threads = row_threads(n);
  const size_t lds = static_cast<size_t>(n) * sizeof(float);
#define LN(TX, TO)                                                                                      \
  layer_norm_kernel<TX, TO><<<count, threads, lds, stream>>>(static_cast<const TX*>(x), w, eps,         \
                                                             static_cast<TO*>(out), rows, n)
  if (x_dtype == TIE_F32 && out_dtype == TIE_F32) LN(float, float);
  else if (x_dtype == TIE_F32 && out_dtype == TIE_BF16) LN(float, bf16_t);
  else if (x_dtype == TIE_BF16 && out_dtype == TIE_BF16) LN(bf16_t, bf16_t);
  else if (x_dtype == TIE_BF16 && out_dtype == TIE_F32) LN(bf16_t, float);
  else return TIE_BAD_ARGUMENT;
#undef LN
  return tie_launch_status();
}

// ------------------------------------------------------------------ hyper-connections
struct HyperWrite {
  const float* y;          // null: no write in this launch
  size_t plane_stride;     // elements between two planes of y
  int planes;
  const float* mix;        // [streams][streams], from x to
  const float* out;        // [streams]
};

struct HyperRead {
  const float* in;         // [streams]; null: no read in this launch
  const float* w;          // the norm's weight
  float eps;
  int norm;                // 0: layer norm, 1: RMS norm, 2: none (h = u as float32)
};

template <typename TO>
__global__ void hyper_connection_kernel(float* __restrict__ streams, size_t stream_stride, int S, int from_x,
                                        float* __restrict__ x, int fold, HyperWrite wr, HyperRead rd,
                                        TO* __restrict__ h, int n) {
  extern __shared__ float urow[];
  __shared__ float scratch[16];
  __shared__ float coef[HYPER_MAX_STREAMS * HYPER_MAX_STREAMS + 2 * HYPER_MAX_STREAMS];
  float* mix = coef;
  float* outw = coef + HYPER_MAX_STREAMS * HYPER_MAX_STREAMS;
  float* inw = outw + HYPER_MAX_STREAMS;
  if (threadIdx.x < S * S && wr.y) mix[threadIdx.x] = wr.mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (wr.y) outw[threadIdx.x] = wr.out[threadIdx.x];
    if (rd.in) inw[threadIdx.x] = rd.in[threadIdx.x];
  }
  __syncthreads();
  const size_t t = blockIdx.x;
  float sum = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const size_t at = t * n + c;
    float old[HYPER_MAX_STREAMS], now[HYPER_MAX_STREAMS];
    if (from_x) {
      const float v = x[at];
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s) old[s] = v;
    } else {
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s) old[s] = s < S ? streams[s * stream_stride + at] : 0.f;
    }
    if (wr.y) {
      float y = 0.f;
      for (int p = 0; p < wr.planes; ++p) y += wr.y[p * wr.plane_stride + at];
#pragma unroll
      for (int to = 0; to < HYPER_MAX_STREAMS; ++to) {
        if (to >= S) break;
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < HYPER_MAX_STREAMS; ++s)
          if (s < S) v = fmaf(mix[s * S + to], old[s], v);
        now[to] = fmaf(outw[to], y, v);
      }
    } else {
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s) now[s] = old[s];
    }
    if (wr.y || from_x) {
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s)
        if (s < S) streams[s * stream_stride + at] = now[s];
    }
    if (fold) {
      float v = 0.f;
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s)
        if (s < S) v += now[s];
      x[at] = v;
    }
    if (rd.in) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s)
        if (s < S) u = fmaf(inw[s], now[s], u);
      urow[c] = u;
      sum += u;
    }
  }
  if (!rd.in) return;
  TO* o = h + t * n;
  if (rd.norm == 2) {
    for (int c = threadIdx.x; c < n; c += blockDim.x) store_from_float(o + c, urow[c]);
    return;
  }
  const float mean = rd.norm == 0 ? block_sum(sum, scratch) / static_cast<float>(n) : 0.f;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float d = urow[c] - mean;
    ss = fmaf(d, d, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + rd.eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x) store_from_float(o + c, ((urow[c] - mean) * inv) * rd.w[c]);
}

// The same pass for rows in steps of four columns (256 to 16384 wide) and up to four streams: a thread holds four
// columns (V times) of every stream in registers, all of a row's loads are under way before the first sum, and the
// row to norm never leaves the registers. Sums run in the order of the kernel above, so both give the same bits.
__device__ __forceinline__ float4 f4_fma(float a, float4 b, float4 c) {
  return make_float4(fmaf(a, b.x, c.x), fmaf(a, b.y, c.y), fmaf(a, b.z, c.z), fmaf(a, b.w, c.w));
}
__device__ __forceinline__ float4 f4_add(float4 a, float4 b) {
  return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}

template <typename TO, int S, int V>
__global__ void hyper_connection_row_kernel(float* __restrict__ streams, size_t stream_stride, int from_x,
                                            float* __restrict__ x, int fold, HyperWrite wr, HyperRead rd,
                                            TO* __restrict__ h, int n) {
  __shared__ float scratch[16];
  const size_t row = static_cast<size_t>(blockIdx.x) * n;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 now[S][V], u[V];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int c = (threadIdx.x + j * blockDim.x) * 4;
    const bool in = c < n;
    const size_t at = row + c;
    float4 old[S];
    if (from_x) {
      const float4 v = in ? *reinterpret_cast<const float4*>(x + at) : zero;
#pragma unroll
      for (int s = 0; s < S; ++s) old[s] = v;
    } else {
#pragma unroll
      for (int s = 0; s < S; ++s) old[s] = in ? *reinterpret_cast<const float4*>(streams + s * stream_stride + at) : zero;
    }
    if (wr.y) {
      float4 y = zero;
      int p = 0;
      if (in) {
        for (; p + 4 <= wr.planes; p += 4) {
          const float4 a = *reinterpret_cast<const float4*>(wr.y + p * wr.plane_stride + at);
          const float4 b = *reinterpret_cast<const float4*>(wr.y + (p + 1) * wr.plane_stride + at);
          const float4 c4 = *reinterpret_cast<const float4*>(wr.y + (p + 2) * wr.plane_stride + at);
          const float4 d = *reinterpret_cast<const float4*>(wr.y + (p + 3) * wr.plane_stride + at);
          y = f4_add(f4_add(f4_add(f4_add(y, a), b), c4), d);
        }
        for (; p < wr.planes; ++p) y = f4_add(y, *reinterpret_cast<const float4*>(wr.y + p * wr.plane_stride + at));
      }
#pragma unroll
      for (int to = 0; to < S; ++to) {
        float4 v = zero;
#pragma unroll
        for (int s = 0; s < S; ++s) v = f4_fma(wr.mix[s * S + to], old[s], v);
        now[to][j] = f4_fma(wr.out[to], y, v);
      }
    } else {
#pragma unroll
      for (int s = 0; s < S; ++s) now[s][j] = old[s];
    }
    if (in && (wr.y || from_x)) {
#pragma unroll
      for (int s = 0; s < S; ++s) *reinterpret_cast<float4*>(streams + s * stream_stride + at) = now[s][j];
    }
    if (in && fold) {
      float4 v = zero;
#pragma unroll
      for (int s = 0; s < S; ++s) v = f4_add(v, now[s][j]);
      *reinterpret_cast<float4*>(x + at) = v;
    }
    u[j] = zero;
    if (rd.in) {
#pragma unroll
      for (int s = 0; s < S; ++s) u[j] = f4_fma(rd.in[s], now[s][j], u[j]);
      sum += (u[j].x + u[j].y) + (u[j].z + u[j].w);
    }
  }
  if (!rd.in) return;
  TO* o = h + row;
  float mean = 0.f, inv = 1.f;
  if (rd.norm != 2) {
    if (rd.norm == 0) mean = block_sum(sum, scratch) / static_cast<float>(n);
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if ((threadIdx.x + j * blockDim.x) * 4 >= n) continue;
      const float a = u[j].x - mean, b = u[j].y - mean, c = u[j].z - mean, d = u[j].w - mean;
      ss += (a * a + b * b) + (c * c + d * d);
    }
    inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + rd.eps);
  }
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int c = (threadIdx.x + j * blockDim.x) * 4;
    if (c >= n) continue;
    float4 w = make_float4(1.f, 1.f, 1.f, 1.f);
    if (rd.norm != 2) w = *reinterpret_cast<const float4*>(rd.w + c);
    store_from_float(o + c, ((u[j].x - mean) * inv) * w.x);
    store_from_float(o + c + 1, ((u[j].y - mean) * inv) * w.y);
    store_from_float(o + c + 2, ((u[j].z - mean) * inv) * w.z);
    store_from_float(o + c + 3, ((u[j].w - mean) * inv) * w.w);
  }
}

template <typename TO, int S>
static void launch_hyper_row(float* streams, size_t stream_stride, int from_x, float* x, int fold, HyperWrite wr,
                             HyperRead rd, TO* h, int T, int n, hipStream_t stream) {
  const int quads = n / 4;
  if (quads <= 1024) {
    const int threads = (quads + TIE_WAVE - 1) / TIE_WAVE * TIE_WAVE;
    hyper_connection_row_kernel<TO, S, 1><<<T, threads, 0, stream>>>(streams, stream_stride, from_x, x, fold, wr, rd, h, n);
  } else if (quads <= 2048) {
    hyper_connection_row_kernel<TO, S, 2><<<T, 1024, 0, stream>>>(streams, stream_stride, from_x, x, fold, wr, rd, h, n);
  } else {
    hyper_connection_row_kernel<TO, S, 4><<<T, 1024, 0, stream>>>(streams, stream_stride, from_x, x, fold, wr, rd, h, n);
  }
}

// streams: [S][T][n] float32. from_x: the streams do not exist yet and all equal x. y (or null) with `planes` planes
// `plane_stride` apart. fold: x <- sum of the (new) streams. in (or null): the next read, normed
// by `norm` (0 layer norm, 1 RMS norm, 2 none) with weight w into h of type h_dtype.
extern "C" int tie_hyper_connection(float* streams, long stream_stride, int S, int from_x, float* x, int fold,
                                    const float* y, long plane_stride, int planes,
                                    const float* mix, const float* out, const float* in, const float* w, float eps,
                                    int norm, void* h, int h_dtype, int T, int n, hipStream_t stream) {
  if (T <= 0 || n <= 0 || S <= 0 || S > HYPER_MAX_STREAMS || planes < 0 ||
      static_cast<size_t>(n) * 4 > 65536)
    return TIE_BAD_ARGUMENT;
  if ((from_x || fold) && !x) return TIE_BAD_ARGUMENT;
  if (y && (!mix || !out || planes < 1)) return TIE_BAD_ARGUMENT;
  if (in && (!h || (norm != 2 && !w))) return TIE_BAD_ARGUMENT;
  HyperWrite wr{y, static_cast<size_t>(plane_stride), planes, mix, out};
  HyperRead rd{in, w, eps, norm};
  if (in && h_dtype != TIE_F32 && h_dtype != TIE_BF16) return TIE_BAD_ARGUMENT;
  if (S <= 4 && n % 4 == 0 && n >= 256 && n <= 16384 && stream_stride % 4 == 0 && (!y || plane_stride % 4 == 0)) {
    const size_t ss = static_cast<size_t>(stream_stride);
#define ROW(TO, COUNT) launch_hyper_row<TO, COUNT>(streams, ss, from_x, x, fold, wr, rd, static_cast<TO*>(h), T, n, stream)
    if (!in || h_dtype == TIE_F32) {
      if (S == 1) ROW(float, 1); else if (S == 2) ROW(float, 2); else if (S == 3) ROW(float, 3); else ROW(float, 4);
    } else {
      if (S == 1) ROW(bf16_t, 1); else if (S == 2) ROW(bf16_t, 2); else if (S == 3) ROW(bf16_t, 3); else ROW(bf16_t, 4);
    }
#undef ROW
    return tie_launch_status();
  }
  const int threads = row_threads(n);
  const size_t lds = in ? static_cast<size_t>(n) * sizeof(float) : 0;
  if (!in || h_dtype == TIE_F32)
    hyper_connection_kernel<float><<<T, threads, lds, stream>>>(streams, static_cast<size_t>(stream_stride), S, from_x,
                                                                x, fold, wr, rd, static_cast<float*>(h), n);
  else if (h_dtype == TIE_BF16)
    hyper_connection_kernel<bf16_t><<<T, threads, lds, stream>>>(streams, static_cast<size_t>(stream_stride), S,
                                                                 from_x, x, fold, wr, rd, static_cast<bf16_t*>(h), n);
  else
    return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}
