// Kernels that work element by element, with no statistics over a row.
//
//   dynamic_tanh   a norm that computes no mean and no variance: out = tanh(alpha * x) * w + b, with a scalar
//                  alpha read on the device and vectors w and b. The stream x is float32; planes of partial sums
//                  still owed to it (a product cut along K) are added first, in plane order, and the sum is
//                  written back, so the pass that reads the stream anyway also settles it. Rows can be gathered
//                  (the head norms only the wanted rows). `plain` leaves out the function: out = x in the
//                  output's type, for a consumer that reads the stream itself. Float32 rows out take the
//                  library's tanhf; rows that are rounded to bfloat16 anyway take tanh on the hardware's 2^x and
//                  reciprocal (float32 arithmetic, absolute error of a few 1e-7).
//   token_gate     out[t][j] = gelu_tanh(gate[t][j]) * table[token[t]][first + j]: a per-token vector out of a
//                  table that all layers share, each with a range of columns of its own, multiplied into a gate
//                  the layer computed from the stream.
#include "common.h"

#include <math.h>

template <typename TO>
__device__ __forceinline__ float tanh_for(float x);
template <>
__device__ __forceinline__ float tanh_for<float>(float x) { return tanhf(x); }
template <>
__device__ __forceinline__ float tanh_for<bf16_t>(float x) { return tanh_fast(x); }

template <typename TO, bool PLAIN>
__global__ void dynamic_tanh_kernel(float* __restrict__ x, const float* __restrict__ partials, size_t plane_stride,
                                    int planes, const float* __restrict__ alpha, const float* __restrict__ w,
                                    const float* __restrict__ b, TO* __restrict__ out, const int* __restrict__ rows,
                                    int n) {
  const size_t r = blockIdx.y;
  const size_t src = rows != nullptr ? static_cast<size_t>(rows[r]) : r;
  const float a = PLAIN ? 0.f : alpha[0];
  for (int i = (blockIdx.x * blockDim.x + threadIdx.x) * 4; i < n; i += gridDim.x * blockDim.x * 4) {
    const size_t at = src * n + i;
    if (i + 3 < n && n % 4 == 0) {
      float4 v = *reinterpret_cast<const float4*>(x + at);
      if (planes > 0) {
        for (int p = 0; p < planes; ++p) {
          const float4 o = *reinterpret_cast<const float4*>(partials + p * plane_stride + at);
          v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
        }
        *reinterpret_cast<float4*>(x + at) = v;
      }
      float y[4] = {v.x, v.y, v.z, v.w};
      if (!PLAIN) {
#pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = fmaf(tanh_for<TO>(a * y[j]), w[i + j], b[i + j]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) store_from_float(out + r * n + i + j, y[j]);
    } else {
      for (int j = 0; j < 4 && i + j < n; ++j) {
        float v = x[at + j];
        if (planes > 0) {
          for (int p = 0; p < planes; ++p) v += partials[p * plane_stride + at + j];
          x[at + j] = v;
        }
        store_from_float(out + r * n + i + j, PLAIN ? v : fmaf(tanh_for<TO>(a * v), w[i + j], b[i + j]));
      }
    }
  }
}

// x float32 [rows of the stream][n]; partials (or null) `planes` planes of the same shape, `plane_stride` floats
// apart, added into x (only without `rows`: a gathered row must not be settled twice). out [R][n] of out_dtype.
extern "C" int tie_dynamic_tanh(float* x, const float* partials, long plane_stride, int planes, const float* alpha,
                                const float* w, const float* b, void* out, int out_dtype, const int* rows, int R, int n,
                                int plain, hipStream_t stream) {
  if (R <= 0 || R > 65535 || n <= 0 || planes < 0 || (planes > 0 && (partials == nullptr || rows != nullptr)) ||
      (!plain && (alpha == nullptr || w == nullptr || b == nullptr)))
    return TIE_BAD_ARGUMENT;
  const int threads = 256;
  const int per_row = (n + 4 * threads - 1) / (4 * threads);
  const dim3 grid(per_row > 64 ? 64 : per_row, R);
#define DT(TO, P)                                                                                             \
  dynamic_tanh_kernel<TO, P><<<grid, threads, 0, stream>>>(x, partials, static_cast<size_t>(plane_stride), planes, \
                                                           alpha, w, b, static_cast<TO*>(out), rows, n)
  if (out_dtype == TIE_F32) { if (plain) DT(float, true); else DT(float, false); }
  else if (out_dtype == TIE_BF16) { if (plain) DT(bf16_t, true); else DT(bf16_t, false); }
  else return TIE_BAD_ARGUMENT;
#undef DT
  return tie_launch_status();
}

template <typename TT, typename TO>
__global__ void token_gate_kernel(const float* __restrict__ gate, const int* __restrict__ tokens,
                                  const TT* __restrict__ table, int table_row, int first, TO* __restrict__ out, int T,
                                  int dim) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<size_t>(T) * dim) return;
  const size_t t = i / dim;
  const int j = static_cast<int>(i % dim);
  const float e = load_as_float(table + static_cast<size_t>(tokens[t]) * table_row + first + j);
  store_from_float(out + i, gelu_tanh_exact(gate[i]) * e);
}

extern "C" int tie_token_gate(const float* gate, const int* tokens, const void* table, int table_dtype, int table_row,
                              int first, void* out, int out_dtype, int T, int dim, hipStream_t stream) {
  if (T <= 0 || dim <= 0 || first < 0 || first + dim > table_row) return TIE_BAD_ARGUMENT;
  const size_t n = static_cast<size_t>(T) * dim;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
#define TG(TT, TO)                                                                                               \
  token_gate_kernel<TT, TO><<<blocks, 256, 0, stream>>>(gate, tokens, static_cast<const TT*>(table), table_row, \
                                                        first, static_cast<TO*>(out), T, dim)
  if (table_dtype == TIE_BF16 && out_dtype == TIE_BF16) TG(bf16_t, bf16_t);
  else if (table_dtype == TIE_F32 && out_dtype == TIE_F32) TG(float, float);
  else if (table_dtype == TIE_BF16 && out_dtype == TIE_F32) TG(bf16_t, float);
  else if (table_dtype == TIE_F32 && out_dtype == TIE_BF16) TG(float, bf16_t);
  else return TIE_BAD_ARGUMENT;
#undef TG
  return tie_launch_status();
}
