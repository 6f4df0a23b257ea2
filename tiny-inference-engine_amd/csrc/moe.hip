// A routed feed-forward (mixture of experts) for gfx950: the router's choice, the rows sorted by expert, and the
// experts' two products over the sorted rows.
//
//   route      scores s = softmax(logits) over all experts of a row, or sigmoid(logits) expert by expert (float32);
//              the choice looks at s + correction: experts form `groups` equal groups of neighbours, a group scores
//              its best member (or the sum of its `group_top` best), only members of the `keep` best groups stay
//              eligible (the others count as -inf), and the `top` best of those are chosen, ties to the lower index;
//              the weights are s at the chosen, as they are or divided by their sum (+ an eps), times a factor.
//              `shared` further slots a row name the experts E, E + 1, ... (experts every row uses: a shared expert,
//              cut into pieces of the routed experts' size), all with the weight sigmoid(logits[E]), one more
//              column of the router's product.
//   align      the T * top (row, choice) slots sorted by expert: offsets[e] .. offsets[e + 1] are the places of
//              expert e's slots, slot_at[place] = slot, where[slot] = place (-1 for a choice >= `real`: an expert
//              without weights, which the caller treats as it likes), and the list of row tiles (expert, first
//              place) the products run over. Integer counters only; which place a slot gets inside its expert's
//              range depends on timing, but no result does: a row's sums are formed the same way at every place.
//   products   act[place] = silu(x[row] Wg_e^T) * (x[row] Wu_e^T), or relu(x[row] Wu_e^T)^2 for experts without a
//              gate, and   parts[place] = act[place] Wd_e^T,
//              one workgroup a (row tile of one expert, column tile). The generic kernels multiply and add in
//              float32 on the vector units for any sizes and float32 / bfloat16 operands (the true 32-bit path);
//              the bfloat16 kernels run the same tiles on the matrix cores.
//
// Nothing here reads the step on the host: the tile list and its length live on the device, the grid is sized
// for the most tiles T * top slots can make and workgroups beyond the list leave at once.
#include "common.h"

#include <math.h>

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_GROUP_TOP 8     // members of a group whose scores make the group's score

// ------------------------------------------------------------------ route
// One wave a row. LDS: the scores, the choice scores, the groups' scores.
__device__ __forceinline__ void wave_argmax(float& v, int& i) {   // ties: the lower index
#pragma unroll
  for (int off = TIE_WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, TIE_WAVE);
    const int oi = __shfl_xor(i, off, TIE_WAVE);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

__global__ __launch_bounds__(TIE_WAVE) void moe_route_kernel(const float* __restrict__ logits, int row,
                                                             const float* __restrict__ correction, int E, int groups,
                                                             int keep, int top, int sigmoid_scores, int group_top,
                                                             int renormalize, float renorm_eps, float weight_scale,
                                                             int shared, int* __restrict__ ids,
                                                             float* __restrict__ weights) {
  extern __shared__ float lds[];
  float* score = lds;              // [E]
  float* choice = score + E;       // [E]
  float* group_score = choice + E; // [groups]
  const int lane = threadIdx.x;
  const size_t t = blockIdx.x;
  const float* z = logits + t * row;
  const int slots = top + shared;          // of a row: the chosen, then the experts every row uses
  if (sigmoid_scores) {
    for (int e = lane; e < E; e += TIE_WAVE) {
      const float s = 1.0f / (1.0f + expf(-z[e]));
      score[e] = s;
      choice[e] = s + (correction != nullptr ? correction[e] : 0.f);
    }
  } else {
    float m = -INFINITY;
    for (int e = lane; e < E; e += TIE_WAVE) m = fmaxf(m, z[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += TIE_WAVE) {
      const float p = expf(z[e] - m);
      score[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += TIE_WAVE) {
      const float s = score[e] / sum;
      score[e] = s;
      choice[e] = s + (correction != nullptr ? correction[e] : 0.f);
    }
  }
  __syncthreads();
  const int size = E / groups;
  if (groups > 1 && keep < groups) {
    for (int g = lane; g < groups; g += TIE_WAVE) {
      // the sum of the group's `group_top` best members (1: its best), the best first; ties to the lower index
      float total = 0.f;
      int taken[MOE_MAX_GROUP_TOP];
      for (int k = 0; k < group_top && k < size; ++k) {
        float best = -INFINITY;
        int at = -1;
        for (int j = 0; j < size; ++j) {
          bool used = false;
          for (int u = 0; u < k; ++u) used = used || taken[u] == j;
          const float v = choice[g * size + j];
          if (!used && (at < 0 || v > best)) {
            best = v;
            at = j;
          }
        }
        taken[k] = at;
        total = k == 0 ? best : total + best;
      }
      group_score[g] = total;
    }
    __syncthreads();
    // the `keep` best groups get +inf as their mark, one at a time
    for (int k = 0; k < keep; ++k) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += TIE_WAVE) {
        const float v = group_score[g];
        if (v != INFINITY && (v > bv || (v == bv && g < bi))) {
          bv = v;
          bi = g;
        }
      }
      wave_argmax(bv, bi);
      if (lane == 0 && bi < groups) group_score[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += TIE_WAVE)
      if (group_score[e / size] != INFINITY) choice[e] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += TIE_WAVE) {
      const float v = choice[e];
      if (v > bv || (v == bv && e < bi && v != -INFINITY)) {
        bv = v;
        bi = e;
      }
    }
    wave_argmax(bv, bi);
    if (bi >= E) bi = 0;               // fewer eligible experts than `top`: a configuration's fault, not a fault here
    if (lane == 0) {
      ids[t * slots + k] = bi;
      weights[t * slots + k] = bv == -INFINITY ? 0.f : score[bi];
      choice[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (lane == 0) {
    float* w = weights + t * slots;
    if (renormalize) {
      float sum = 0.f;
      for (int k = 0; k < top; ++k) sum += w[k];
      sum += renorm_eps;
      for (int k = 0; k < top; ++k) w[k] = w[k] / sum * weight_scale;
    } else if (weight_scale != 1.0f) {
      for (int k = 0; k < top; ++k) w[k] *= weight_scale;
    }
    if (shared > 0) {
      const float g = 1.0f / (1.0f + expf(-z[E]));
      for (int k = 0; k < shared; ++k) {
        ids[t * slots + top + k] = E + k;
        w[top + k] = g;
      }
    }
  }
}

// logits [T][row] float32 with row >= E (+ 1 with shared slots: column E is the gate of the experts every row uses);
// ids and weights [T][top + shared].
extern "C" int tie_moe_route(const float* logits, int row, const float* correction, int T, int E, int groups, int keep,
                             int top, int sigmoid_scores, int group_top, int renormalize, float renorm_eps,
                             float weight_scale, int shared, int* ids, float* weights, hipStream_t stream) {
  if (T <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || groups <= 0 || E % groups != 0 || keep <= 0 || keep > groups ||
      top <= 0 || top > E || group_top <= 0 || group_top > MOE_MAX_GROUP_TOP || shared < 0 ||
      row < E + (shared > 0 ? 1 : 0))
    return TIE_BAD_ARGUMENT;
  const size_t lds = sizeof(float) * (2 * static_cast<size_t>(E) + groups);
  moe_route_kernel<<<T, TIE_WAVE, lds, stream>>>(logits, row, correction, E, groups, keep, top, sigmoid_scores,
                                                 group_top, renormalize, renorm_eps, weight_scale, shared, ids,
                                                 weights);
  return tie_launch_status();
}

// ------------------------------------------------------------------ align
#define ALIGN_THREADS 1024

__global__ __launch_bounds__(ALIGN_THREADS) void moe_align_kernel(const int* __restrict__ ids, int slots, int real,
                                                                  int tile_rows, int* __restrict__ offsets,
                                                                  int* __restrict__ slot_at, int* __restrict__ where,
                                                                  int* __restrict__ tiles, int max_tiles,
                                                                  int* __restrict__ num_tiles) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int cursor[MOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  for (int e = tid; e < real; e += ALIGN_THREADS) count[e] = 0;
  __syncthreads();
  for (int s = tid; s < slots; s += ALIGN_THREADS) {
    const int e = ids[s];
    if (e >= 0 && e < real) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0, n = 0;
    for (int e = 0; e < real; ++e) {
      offsets[e] = at;
      cursor[e] = at;
      for (int r = 0; r < count[e] && n < max_tiles; r += tile_rows, ++n) {
        tiles[2 * n] = e;
        tiles[2 * n + 1] = at + r;
      }
      at += count[e];
    }
    offsets[real] = at;
    *num_tiles = n;
  }
  __syncthreads();
  for (int s = tid; s < slots; s += ALIGN_THREADS) {
    const int e = ids[s];
    if (e >= 0 && e < real) {
      const int place = atomicAdd(&cursor[e], 1);
      slot_at[place] = s;
      where[s] = place;
    } else {
      where[s] = -1;
    }
  }
}

// The most row tiles `slots` slots over `real` experts can make: every expert's last tile may be ragged.
extern "C" int tie_moe_max_tiles(int slots, int real, int tile_rows) {
  if (slots <= 0 || real <= 0 || tile_rows <= 0) return 0;
  return slots / tile_rows + (real < slots ? real : slots);
}

extern "C" int tie_moe_align(const int* ids, int slots, int real, int tile_rows, int* offsets, int* slot_at, int* where,
                             int* tiles, int max_tiles, int* num_tiles, hipStream_t stream) {
  if (slots <= 0 || real <= 0 || real > MOE_MAX_EXPERTS || tile_rows <= 0 ||
      max_tiles < tie_moe_max_tiles(slots, real, tile_rows))
    return TIE_BAD_ARGUMENT;
  moe_align_kernel<<<1, ALIGN_THREADS, 0, stream>>>(ids, slots, real, tile_rows, offsets, slot_at, where, tiles,
                                                    max_tiles, num_tiles);
  return tie_launch_status();
}

// ------------------------------------------------------------------ products, float32 arithmetic
// Tiles of GR rows x GC columns, k staged GK at a time; a thread sums 2 x 4 outputs over k in ascending order.
#define GR 32
#define GC 64
#define GK 16

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }

// MODE 1 (gated): x rows are gathered (row = slot_at[place] / top), w_a and w_b are the gate and up weights
// [real][N][K], out[place][c] = silu(a) * b. MODE 2 (experts without a gate): rows gathered likewise, w_a the up
// weight, out[place][c] = relu(a)^2. MODE 0: x rows are the places themselves (act [slots][K]), w_a is the down
// weight and out[place][c] = a.
__device__ __forceinline__ float relu_squared_f(float a) { const float r = fmaxf(a, 0.f); return r * r; }

template <typename TX, typename TW, typename TO, int MODE>
__global__ __launch_bounds__(256) void moe_gemm_generic_kernel(
    const TX* __restrict__ x, const TW* __restrict__ w_a, const TW* __restrict__ w_b, TO* __restrict__ out,
    const int* __restrict__ offsets, const int* __restrict__ slot_at, const int* __restrict__ tiles,
    const int* __restrict__ num_tiles, int top, int N, int K) {
  constexpr bool GATED = MODE == 1;
  constexpr bool GATHER = MODE != 0;
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  __shared__ float xs[GK][GR + 4];
  __shared__ float as[GK][GC + 4];
  __shared__ float bs[GATED ? GK : 1][GC + 4];
  __shared__ int src[GR];
  const int e = tiles[2 * tile];
  const int place0 = tiles[2 * tile + 1];
  const int rows = min(GR, offsets[e + 1] - place0);
  const int col0 = blockIdx.y * GC;
  const int tid = threadIdx.x;
  if (tid < GR) src[tid] = tid < rows ? (GATHER ? slot_at[place0 + tid] / top : place0 + tid) : -1;
  __syncthreads();
  const TW* wa = w_a + static_cast<size_t>(e) * N * K;
  const TW* wb = GATED ? w_b + static_cast<size_t>(e) * N * K : nullptr;
  const int ty = tid / 16, tx = tid % 16;      // rows ty * 2 + {0, 1}, columns tx * 4 + {0..3}
  float acc_a[2][4], acc_b[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc_a[i][j] = acc_b[i][j] = 0.f;
  const int lr = tid / 4;          // 0..63
  const int lk = (tid % 4) * 4;    // 0, 4, 8, 12
  for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      if (lr < GR) {
        const int r = src[lr];
        xs[lk + i][lr] = (r >= 0 && k < K) ? load_as_float(x + static_cast<size_t>(r) * K + k) : 0.f;
      }
      const int c = col0 + lr;
      as[lk + i][lr] = (c < N && k < K) ? load_as_float(wa + static_cast<size_t>(c) * K + k) : 0.f;
      if (GATED) bs[lk + i][lr] = (c < N && k < K) ? load_as_float(wb + static_cast<size_t>(c) * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      float xv[2], av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) xv[i] = xs[k][ty * 2 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        av[j] = as[k][tx * 4 + j];
        bv[j] = GATED ? bs[k][tx * 4 + j] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc_a[i][j] = fmaf(xv[i], av[j], acc_a[i][j]);
          if (GATED) acc_b[i][j] = fmaf(xv[i], bv[j], acc_b[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = ty * 2 + i;
    if (r >= rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c >= N) continue;
      const float v = GATED ? silu_f(acc_a[i][j]) * acc_b[i][j]
                            : (MODE == 2 ? relu_squared_f(acc_a[i][j]) : acc_a[i][j]);
      store_from_float(out + static_cast<size_t>(place0 + r) * N + c, v);
    }
  }
}

extern "C" int tie_moe_generic_tile_rows() { return GR; }

// gated = 1: out [slots][N] of out_dtype = silu(x Wa^T) * (x Wb^T) over gathered rows of x [T][K];
// gated = 2: out [slots][N] of out_dtype = relu(x Wa^T)^2 over gathered rows of x [T][K];
// gated = 0: out [slots][N] = x Wa^T over x [slots][K]. Weights [real][N][K].
extern "C" int tie_moe_gemm_generic(const void* x, int x_dtype, const void* w_a, const void* w_b, int w_dtype, void* out,
                                    int out_dtype, int gated, const int* offsets, const int* slot_at, const int* tiles,
                                    const int* num_tiles, int max_tiles, int top, int N, int K, hipStream_t stream) {
  if (max_tiles <= 0 || top <= 0 || N <= 0 || K <= 0 || gated < 0 || gated > 2 || (gated == 1 && w_b == nullptr))
    return TIE_BAD_ARGUMENT;
  if ((x_dtype | w_dtype | out_dtype) & ~1) return TIE_BAD_ARGUMENT;
  const dim3 grid(max_tiles, (N + GC - 1) / GC);
  if (grid.y > 65535) return TIE_BAD_ARGUMENT;
#define LAUNCH_G(TX, TW, TO, G)                                                                                    \
  moe_gemm_generic_kernel<TX, TW, TO, G><<<grid, 256, 0, stream>>>(                                                \
      static_cast<const TX*>(x), static_cast<const TW*>(w_a), static_cast<const TW*>(w_b), static_cast<TO*>(out), \
      offsets, slot_at, tiles, num_tiles, top, N, K)
#define LAUNCH(TX, TW, TO)                    \
  {                                           \
    if (gated == 1) LAUNCH_G(TX, TW, TO, 1);  \
    else if (gated == 2) LAUNCH_G(TX, TW, TO, 2); \
    else LAUNCH_G(TX, TW, TO, 0);             \
  }
  const int key = x_dtype * 4 + w_dtype * 2 + out_dtype;
  switch (key) {
    case 0: LAUNCH(float, float, float) break;
    case 2: LAUNCH(float, bf16_t, float) break;
    case 6: LAUNCH(bf16_t, bf16_t, float) break;
    case 7: LAUNCH(bf16_t, bf16_t, bf16_t) break;
    default: return TIE_BAD_ARGUMENT;
  }
#undef LAUNCH
#undef LAUNCH_G
  return tie_launch_status();
}

// ------------------------------------------------------------------ products on the matrix cores (bfloat16)
// v_mfma_f32_16x16x32_bf16 with the weights as the A operand (16 weight rows) and the rows of x as B (16 rows of
// a tile): lane l gives 8 consecutive k (k0 + 8 (l / 16) ...) of weight row l % 16 and of x row l % 16, and
// receives the sums of x row l % 16 against weight rows 4 (l / 16) + 0..3. A workgroup of four waves takes one
// row tile of one expert and 64 NT columns, 16 NT a wave.
//   MT = 1, NT = 1: the few rows of decode steps. 16 rows a tile and 16 columns a workgroup, whose four waves
//     take every fourth k-block each and add their sums through LDS in wave order: many small workgroups even
//     where a step uses four experts, every operand from global memory straight into its fragment (16 bytes a
//     lane). With a wave a column tile over all of K (64 columns a workgroup) a batch-1 step's gate/up product over
//     2048 x 768 experts took 31.8 us; so it takes 13.7.
//   MT = 4 or 8 (NT = 4, or 2 for the gated product of MT = 8, whose accumulators are two sets): where an expert
//     has many rows. 64 or 128 rows a tile; a weight fragment meets MT x fragments before it leaves the
//     registers, and the four waves, which all need the same x fragments, load MT / 4 each (a k-block ahead)
//     and pass them round through LDS, two buffers taking turns, one barrier a k-block.
// K in steps of 8 (16-byte pieces); a ragged last block of 32 is filled with zeros. Rows beyond a tile's end
// and columns beyond N are computed on clamped addresses and not stored. A row's sums do not depend on its
// place in the tile.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float moe_floatx4;
typedef uint32_t moe_u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ moe_bf16x8_t moe_frag(moe_u32x4_t v) { return *reinterpret_cast<const moe_bf16x8_t*>(&v); }

__device__ __forceinline__ moe_u32x4_t moe_load8(const bf16_t* p, bool in_range) {
  return in_range ? *reinterpret_cast<const moe_u32x4_t*>(p) : moe_u32x4_t{0u, 0u, 0u, 0u};
}

template <int MT, int NT, int MODE>
__global__ __launch_bounds__(256) void moe_gemm_bf16_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w_a, const bf16_t* __restrict__ w_b,
    void* __restrict__ out, const int* __restrict__ offsets, const int* __restrict__ slot_at,
    const int* __restrict__ tiles, const int* __restrict__ num_tiles, int top, int N, int K) {
  static_assert(MT == 1 || MT == 4 || MT == 8, "one x tile a wave, or MT / 4 loaded by each of the four waves");
  constexpr bool GATED = MODE == 1;       // two weights, silu(a) * b
  constexpr bool GATHER = MODE != 0;      // rows of x gathered by slot; the activations go out as bfloat16
  constexpr int OWN = MT == 1 ? 1 : MT / 4;                  // x fragments this wave loads a k-block
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;                            // the whole workgroup leaves
  constexpr bool KSPLIT = MT == 1;                            // the four waves share the columns and split K
  __shared__ moe_u32x4_t xs[MT > 1 ? 2 : 1][MT][TIE_WAVE];
  __shared__ moe_floatx4 sums[KSPLIT ? 2 : 1][KSPLIT ? 4 : 1][TIE_WAVE];
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int wave = threadIdx.x / TIE_WAVE;
  const int r16 = lane & 15, quad = lane >> 4;
  const int e = tiles[2 * tile];
  const int place0 = tiles[2 * tile + 1];
  const int rows = min(16 * MT, offsets[e + 1] - place0);
  const int col0 = (KSPLIT ? blockIdx.y : blockIdx.y * 4 + wave) * 16 * NT;
  const int k_first = KSPLIT ? wave * 32 : 0;                // this wave's k-blocks: k_first, k_first + k_step, ...
  constexpr int k_step = KSPLIT ? 128 : 32;
  // The x rows this lane loads: with MT = 4 those of the wave's own 16-row tile (clamped to the tile's first row
  // beyond its end: computed, never stored).
  const bf16_t* xr[OWN];
#pragma unroll
  for (int o = 0; o < OWN; ++o) {
    const int own_row = (MT == 1 ? 0 : wave * OWN + o) * 16 + r16;
    const int own_place = place0 + (own_row < rows ? own_row : 0);
    const size_t src = GATHER ? static_cast<size_t>(slot_at[own_place] / top) : static_cast<size_t>(own_place);
    xr[o] = x + src * K + quad * 8;
  }
  const bf16_t* wa[NT];
  const bf16_t* wb[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = min(col0 + nt * 16 + r16, N - 1);
    wa[nt] = w_a + (static_cast<size_t>(e) * N + n) * K + quad * 8;
    wb[nt] = GATED ? w_b + (static_cast<size_t>(e) * N + n) * K + quad * 8 : nullptr;
  }
  moe_floatx4 acc_a[MT][NT], acc_b[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc_a[mt][nt] = acc_b[mt][nt] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
  moe_u32x4_t ahead[OWN];
#pragma unroll
  for (int o = 0; o < OWN; ++o) ahead[o] = moe_load8(xr[o] + k_first, k_first + quad * 8 < K);
  // The weights too are asked for a k-block ahead: a barrier stands in every k-block of the tiles that share x,
  // and loads do not move across it by themselves.
  moe_u32x4_t a_ahead[NT], b_ahead[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    a_ahead[nt] = moe_load8(wa[nt] + k_first, k_first + quad * 8 < K);
    if (GATED) b_ahead[nt] = moe_load8(wb[nt] + k_first, k_first + quad * 8 < K);
  }
#pragma unroll 2
  for (int k0 = k_first; k0 < K; k0 += k_step) {
    const bool next_in_range = k0 + k_step + quad * 8 < K;
    moe_u32x4_t xf[MT], af[NT], bf[NT];
    if constexpr (MT > 1) {
#pragma unroll
      for (int o = 0; o < OWN; ++o) xs[(k0 >> 5) & 1][wave * OWN + o][lane] = ahead[o];
    } else {
      xf[0] = ahead[0];
    }
    if (k0 + k_step < K) {
#pragma unroll
      for (int o = 0; o < OWN; ++o) ahead[o] = moe_load8(xr[o] + k0 + k_step, next_in_range);
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      af[nt] = a_ahead[nt];
      if (GATED) bf[nt] = b_ahead[nt];
    }
    if (k0 + k_step < K) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        a_ahead[nt] = moe_load8(wa[nt] + k0 + k_step, next_in_range);
        if (GATED) b_ahead[nt] = moe_load8(wb[nt] + k0 + k_step, next_in_range);
      }
    }
    if constexpr (MT > 1) {
      __syncthreads();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[mt] = xs[(k0 >> 5) & 1][mt][lane];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc_a[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_frag(af[nt]), moe_frag(xf[mt]), acc_a[mt][nt], 0, 0, 0);
        if (GATED)
          acc_b[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_frag(bf[nt]), moe_frag(xf[mt]), acc_b[mt][nt], 0, 0, 0);
      }
  }
  if constexpr (KSPLIT) {
    static_assert(!KSPLIT || NT == 1, "the waves that split K share one column tile");
    sums[0][wave][lane] = acc_a[0][0];
    if (GATED) sums[1][wave][lane] = acc_b[0][0];
    __syncthreads();
    if (wave != 0) return;
    acc_a[0][0] = sums[0][0][lane];
    if (GATED) acc_b[0][0] = sums[1][0][lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) {                            // in wave order, whatever finished first
      acc_a[0][0] += sums[0][w][lane];
      if (GATED) acc_b[0][0] += sums[1][w][lane];
    }
  }
  // lane: x row mt * 16 + r16, columns col0 + nt * 16 + quad * 4 + 0..3
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + r16;
    if (r >= rows) continue;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int c = col0 + nt * 16 + quad * 4;
      if (c >= N) continue;
      const size_t at = static_cast<size_t>(place0 + r) * N + c;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = GATED ? silu_f(acc_a[mt][nt][i]) * acc_b[mt][nt][i]
                     : (MODE == 2 ? relu_squared_f(acc_a[mt][nt][i]) : acc_a[mt][nt][i]);
      if (GATHER) {
        bf16_t* o = static_cast<bf16_t*>(out) + at;
        if (c + 3 < N && N % 4 == 0) {
          uint2 packed = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          *reinterpret_cast<uint2*>(o) = packed;
        } else {
          for (int i = 0; i < 4; ++i)
            if (c + i < N) o[i] = float_to_bf16(v[i]);
        }
      } else {
        float* o = static_cast<float*>(out) + at;
        if (c + 3 < N && N % 4 == 0) {
          *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
          for (int i = 0; i < 4; ++i)
            if (c + i < N) o[i] = v[i];
        }
      }
    }
  }
}

// Rows of a row tile by the average number of rows an expert gets: 64 or 128 where that fills most of such a tile.
extern "C" int tie_moe_bf16_tile_rows(int slots, int real) {
  return slots >= 96L * real ? 128 : (slots >= 48L * real ? 64 : 16);
}

// bfloat16 x and weights; gated = 1: out bfloat16 [slots][N] = silu(x Wa^T) * (x Wb^T) over gathered rows of x;
// gated = 2: out bfloat16 [slots][N] = relu(x Wa^T)^2 over gathered rows of x;
// gated = 0: out float32 [slots][N] = x Wa^T over x [slots][K]. tile_rows (16, 64 or 128) as given to tie_moe_align.
extern "C" int tie_moe_gemm_bf16(const void* x, const void* w_a, const void* w_b, void* out, int gated,
                                 const int* offsets, const int* slot_at, const int* tiles, const int* num_tiles,
                                 int max_tiles, int tile_rows, int top, int N, int K, hipStream_t stream) {
  if (max_tiles <= 0 || top <= 0 || N <= 0 || K <= 0 || K % 8 != 0 || gated < 0 || gated > 2 ||
      (gated == 1 && w_b == nullptr) || (tile_rows != 16 && tile_rows != 64 && tile_rows != 128) || reinterpret_cast<uintptr_t>(x) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(w_a) % 16 != 0 || reinterpret_cast<uintptr_t>(w_b) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(out) % 16 != 0)
    return TIE_BAD_ARGUMENT;
  const int columns = tile_rows == 16 ? 16 : (tile_rows == 128 && gated == 1 ? 128 : 256);   // of a workgroup
  const dim3 grid(max_tiles, (N + columns - 1) / columns);
  if (grid.y > 65535) return TIE_BAD_ARGUMENT;
#define LAUNCH_B(MT, NT, G)                                                                                  \
  moe_gemm_bf16_kernel<MT, NT, G><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(x),                   \
                                                            static_cast<const bf16_t*>(w_a),                 \
                                                            static_cast<const bf16_t*>(w_b), out, offsets,   \
                                                            slot_at, tiles, num_tiles, top, N, K)
  if (tile_rows == 128) {
    if (gated == 1) LAUNCH_B(8, 2, 1); else if (gated == 2) LAUNCH_B(8, 4, 2); else LAUNCH_B(8, 4, 0);
  } else if (tile_rows == 64) {
    if (gated == 1) LAUNCH_B(4, 4, 1); else if (gated == 2) LAUNCH_B(4, 4, 2); else LAUNCH_B(4, 4, 0);
  } else {
    if (gated == 1) LAUNCH_B(1, 1, 1); else if (gated == 2) LAUNCH_B(1, 1, 2); else LAUNCH_B(1, 1, 0);
  }
#undef LAUNCH_B
  return tie_launch_status();
}

// ------------------------------------------------------------------ combine
// out[t] (+)= sum over k < top of weights[t][k] * (where[t][k] >= 0 ? parts[where[t][k]] : self[t]) in the order of k.
template <typename TS>
__global__ void moe_combine_kernel(const float* __restrict__ parts, const int* __restrict__ where,
                                   const float* __restrict__ weights, const TS* __restrict__ self,
                                   float* __restrict__ out, int top, int n, int accumulate) {
  const size_t t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float y = 0.f;
  for (int k = 0; k < top; ++k) {
    const int at = where[t * top + k];
    const float part = at >= 0 ? parts[static_cast<size_t>(at) * n + i] : load_as_float(self + t * n + i);
    y = fmaf(weights[t * top + k], part, y);
  }
  out[t * n + i] = accumulate ? out[t * n + i] + y : y;
}

extern "C" int tie_moe_combine(const float* parts, const int* where, const float* weights, const void* self,
                               int self_dtype, float* out, int T, int top, int n, int accumulate,
                               hipStream_t stream) {
  if (T <= 0 || T > 65535 || top <= 0 || n <= 0) return TIE_BAD_ARGUMENT;
  const dim3 grid((n + 255) / 256, T);
  if (self_dtype == TIE_F32)
    moe_combine_kernel<float><<<grid, 256, 0, stream>>>(parts, where, weights, static_cast<const float*>(self), out,
                                                        top, n, accumulate);
  else if (self_dtype == TIE_BF16)
    moe_combine_kernel<bf16_t><<<grid, 256, 0, stream>>>(parts, where, weights, static_cast<const bf16_t*>(self), out,
                                                         top, n, accumulate);
  else
    return TIE_BAD_ARGUMENT;
  return tie_launch_status();
}
