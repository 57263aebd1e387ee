// A feed-forward of routed experts: every token is sent to `top` of `experts` small gated feed-forwards and
// receives the weighted sum of their outputs.
//
//   router_choose     from float32 router logits z: s = sigmoid(z); the `top` experts with the largest s + correction
//                     are chosen (ties: the lower index); a chosen expert's weight is its s, or s divided by the
//                     chosen experts' sum when `renormalize` is set
//   experts_gate_up   for every (token, choice): act = f(W_gate[e] x) * (W_up[e] x), W stored [experts, 2 ff, width]
//   experts_down      y[t] = sum over the token's choices, in their order, of weight * W_down[e] act
//
// The last two read an expert's rows once per (token, choice): the form for steps of few tokens.  Every sum runs in a
// fixed order over a token's own data, so a token's result does not depend on what else is in the batch.
#include "common.h"

__global__ void router_choose_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                     int* __restrict__ ids, float* __restrict__ weights, int tokens, int experts,
                                     int top, int renormalize) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= tokens) return;
  const float* z = logits + (size_t)t * experts;
  int* mine = ids + (size_t)t * top;
  float* w = weights + (size_t)t * top;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float best_score = -INFINITY, best_s = 0.f;
    for (int e = 0; e < experts; ++e) {
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= (mine[j] == e);
      if (taken) continue;
      const float s = 1.f / (1.f + expf(-z[e]));
      const float score = s + (correction ? correction[e] : 0.f);
      if (best < 0 || score > best_score) {
        best = e;
        best_score = score;
        best_s = s;
      }
    }
    mine[k] = best;
    w[k] = best_s;
    total += best_s;
  }
  if (renormalize)
    for (int k = 0; k < top; ++k) w[k] /= total;
}

// A wave per token: lane l holds the scores of experts l, l + 64, ... (up to 8 of them, so up to 512 experts); each
// of the `top` rounds is a maximum over the wave of (choice score, lower index first).
constexpr int kRouterPerLane = 8;

__global__ void __launch_bounds__(256)
router_choose_wave_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                          int* __restrict__ ids, float* __restrict__ weights, int tokens, int experts, int top,
                          int renormalize) {
  const int t = blockIdx.x * 4 + threadIdx.x / kWave;
  if (t >= tokens) return;
  const int lane = threadIdx.x % kWave;
  float score[kRouterPerLane], plain[kRouterPerLane];
#pragma unroll
  for (int j = 0; j < kRouterPerLane; ++j) {
    const int e = lane + j * kWave;
    if (e < experts) {
      plain[j] = 1.f / (1.f + expf(-logits[(size_t)t * experts + e]));
      score[j] = plain[j] + (correction ? correction[e] : 0.f);
    } else {
      plain[j] = 0.f;
      score[j] = -INFINITY;
    }
  }
  float total = 0.f, mine = 0.f;   // lane k keeps the weight of choice k (top <= 64)
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, best_plain = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < kRouterPerLane; ++j)
      if (score[j] > best) {
        best = score[j];
        best_plain = plain[j];
        best_e = lane + j * kWave;
      }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, kWave), op = __shfl_xor(best_plain, off, kWave);
      const int oe = __shfl_xor(best_e, off, kWave);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_plain = op;
        best_e = oe;
      }
    }
#pragma unroll
    for (int j = 0; j < kRouterPerLane; ++j)
      if (lane + j * kWave == best_e) score[j] = -INFINITY;
    if (lane == 0) ids[(size_t)t * top + k] = best_e;
    if (lane == k) mine = best_plain;
    total += best_plain;
  }
  if (lane < top) weights[(size_t)t * top + lane] = renormalize ? mine / total : mine;
}

ATOM_EXPORT int atom_router_choose(const float* logits, const float* correction, int* ids, float* weights, int tokens,
                                   int experts, int top, int renormalize, hipStream_t stream) {
  if (tokens < 0 || experts <= 0 || top <= 0 || top > experts) return ATOM_BAD_SHAPE;
  if (logits == nullptr || ids == nullptr || weights == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  if (experts <= kRouterPerLane * kWave && top <= kWave) {
    hipLaunchKernelGGL(router_choose_wave_kernel, dim3((tokens + 3) / 4), dim3(256), 0, stream, logits, correction, ids,
                       weights, tokens, experts, top, renormalize);
    return launch_status();
  }
  hipLaunchKernelGGL(router_choose_kernel, dim3((tokens + 127) / 128), dim3(128), 0, stream, logits, correction, ids,
                     weights, tokens, experts, top, renormalize);
  return launch_status();
}

__device__ __forceinline__ float expert_activation(float g, int act) {
  if (act == 1) return g > 0.f ? g : 0.f;
  if (act == 2) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  return g / (1.f + expf(-g));
}

constexpr int kExpCols = 32;   // output columns of a block: 4 waves x 8
typedef __attribute__((ext_vector_type(8))) __bf16 ex_bf16x8;

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
experts_gate_up_kernel(const T* __restrict__ x, const TW* __restrict__ w, const int* __restrict__ ids,
                       T* __restrict__ act_out, int top, int ff, int width, int act) {
  extern __shared__ float xs[];   // width
  const int pair = blockIdx.x;
  const int t = pair / top;
  const int e = ids[pair];
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const T* xr = x + (size_t)t * width;
  for (int i = tid; i < width; i += 256) xs[i] = to_f32(xr[i]);
  __syncthreads();
  const TW* we = w + (size_t)e * 2 * ff * width;
  for (int c = 0; c < kExpCols / 4; ++c) {
    const int col = blockIdx.y * kExpCols + wave * (kExpCols / 4) + c;
    if (col >= ff) break;
    const TW* gr = we + (size_t)col * width;
    const TW* ur = we + (size_t)(ff + col) * width;
    float g = 0.f, u = 0.f;
    if constexpr (sizeof(TW) == 2) {
      if (width % 8 == 0) {   // 16 bytes a lane and row
        for (int i = lane * 8; i < width; i += kWave * 8) {
          const ex_bf16x8 gv = *reinterpret_cast<const ex_bf16x8*>(gr + i), uv = *reinterpret_cast<const ex_bf16x8*>(ur + i);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            g = fmaf(xs[i + e], static_cast<float>(gv[e]), g);
            u = fmaf(xs[i + e], static_cast<float>(uv[e]), u);
          }
        }
      } else {
        for (int i = lane; i < width; i += kWave) {
          g = fmaf(xs[i], to_f32(gr[i]), g);
          u = fmaf(xs[i], to_f32(ur[i]), u);
        }
      }
    } else {
      for (int i = lane; i < width; i += kWave) {
        const float xv = xs[i];
        g = fmaf(xv, to_f32(gr[i]), g);
        u = fmaf(xv, to_f32(ur[i]), u);
      }
    }
    g = wave_sum(g);
    u = wave_sum(u);
    if (lane == 0) act_out[(size_t)pair * ff + col] = from_f32<T>(expert_activation(g, act) * u);
  }
}

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
experts_down_kernel(const T* __restrict__ act_in, const TW* __restrict__ w, const int* __restrict__ ids,
                    const float* __restrict__ weights, T* __restrict__ y, int top, int ff, int width) {
  extern __shared__ float as[];   // top * ff
  const int t = blockIdx.x;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  for (int i = tid; i < top * ff; i += 256) as[i] = to_f32(act_in[(size_t)t * top * ff + i]);
  __syncthreads();
  for (int c = 0; c < kExpCols / 4; ++c) {
    const int col = blockIdx.y * kExpCols + wave * (kExpCols / 4) + c;
    if (col >= width) break;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
      const int e = ids[(size_t)t * top + k];
      const TW* wr = w + ((size_t)e * width + col) * ff;
      float s = 0.f;
      bool done = false;
      if constexpr (sizeof(TW) == 2) {
        if (ff % 8 == 0) {
          for (int i = lane * 8; i < ff; i += kWave * 8) {
            const ex_bf16x8 wv = *reinterpret_cast<const ex_bf16x8*>(wr + i);
#pragma unroll
            for (int e = 0; e < 8; ++e) s = fmaf(as[k * ff + i + e], static_cast<float>(wv[e]), s);
          }
          done = true;
        }
      }
      if (!done)
        for (int i = lane; i < ff; i += kWave) s = fmaf(as[k * ff + i], to_f32(wr[i]), s);
      total += weights[(size_t)t * top + k] * wave_sum(s);
    }
    if (lane == 0) y[(size_t)t * width + col] = from_f32<T>(total);
  }
}

ATOM_EXPORT int atom_experts_gate_up(const void* x, const void* w, int w_dtype, const int* ids, void* act_out, int dtype,
                                     int tokens, int top, int ff, int width, int act, hipStream_t stream) {
  if (tokens < 0 || top <= 0 || ff <= 0 || width <= 0 || act < 0 || act > 2) return ATOM_BAD_SHAPE;
  if (x == nullptr || w == nullptr || ids == nullptr || act_out == nullptr) return ATOM_BAD_SHAPE;
  if ((size_t)width * sizeof(float) > 64 * 1024) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  dim3 grid(tokens * top, (ff + kExpCols - 1) / kExpCols), block(256);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
  const size_t smem = (size_t)width * sizeof(float);
#define LAUNCH(T, TW)                                                                                              \
  hipLaunchKernelGGL((experts_gate_up_kernel<T, TW>), grid, block, smem, stream, (const T*)x, (const TW*)w, ids, \
                     (T*)act_out, top, ff, width, act)
  if (dtype == ATOM_F32 && w_dtype == ATOM_F32) LAUNCH(float, float);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_BF16) LAUNCH(bf16_t, bf16_t);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_F32) LAUNCH(bf16_t, float);
  else return ATOM_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

ATOM_EXPORT int atom_experts_down(const void* act_in, const void* w, int w_dtype, const int* ids, const float* weights,
                                  void* y, int dtype, int tokens, int top, int ff, int width, hipStream_t stream) {
  if (tokens < 0 || top <= 0 || ff <= 0 || width <= 0) return ATOM_BAD_SHAPE;
  if (act_in == nullptr || w == nullptr || ids == nullptr || weights == nullptr || y == nullptr) return ATOM_BAD_SHAPE;
  if ((size_t)top * ff * sizeof(float) > 64 * 1024) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  dim3 grid(tokens, (width + kExpCols - 1) / kExpCols), block(256);
  if (grid.y > 65535) return ATOM_TOO_LARGE;
  const size_t smem = (size_t)top * ff * sizeof(float);
#define LAUNCH(T, TW)                                                                                               \
  hipLaunchKernelGGL((experts_down_kernel<T, TW>), grid, block, smem, stream, (const T*)act_in, (const TW*)w, ids, \
                     weights, (T*)y, top, ff, width)
  if (dtype == ATOM_F32 && w_dtype == ATOM_F32) LAUNCH(float, float);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_BF16) LAUNCH(bf16_t, bf16_t);
  else if (dtype == ATOM_BF16 && w_dtype == ATOM_F32) LAUNCH(bf16_t, float);
  else return ATOM_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// ------------------------------------------------------------------ many tokens: pairs sorted by expert, grouped products
//
//   experts_sort      one block: counts the pairs of every expert, gives each expert whole tiles of 64 rows
//                     (padded), and every pair its row.  tile_expert[tile] = expert or -1; row_pair[row] = pair or
//                     -1; pair_row[pair] = row.  Rows of one expert come in no fixed order; a row's result does
//                     not depend on its place.
//   grouped_gate_up   act[row] = f(W_gate[e] x) * (W_up[e] x) for the rows of a tile, on the matrix cores.  The
//                     weights are the A operand and the tokens the B operand, both read straight from memory in
//                     16-byte pieces, so a lane ends up with four consecutive columns of one row.
//   grouped_down      y[row] = W_down[e] act[row], float32
//   experts_combine   out[t] = sum_k weight[t, k] * y[pair_row[t, k]], in the order of k
//
// bfloat16 only; width and ff multiples of 8.

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

constexpr int kTileRows = 64;

__global__ void __launch_bounds__(1024)
experts_sort_kernel(const int* __restrict__ ids, int pairs, int experts, int max_tiles, int* __restrict__ tile_expert,
                    int* __restrict__ row_pair, int* __restrict__ pair_row) {
  extern __shared__ int sm[];   // counts [experts], first row of each expert [experts]
  int* counts = sm;
  int* first = sm + experts;
  const int tid = threadIdx.x;
  for (int e = tid; e < experts; e += 1024) counts[e] = 0;
  for (int i = tid; i < max_tiles; i += 1024) tile_expert[i] = -1;
  for (int i = tid; i < max_tiles * kTileRows; i += 1024) row_pair[i] = -1;
  __syncthreads();
  for (int i = tid; i < pairs; i += 1024) atomicAdd(&counts[ids[i]], 1);
  __syncthreads();
  if (tid == 0) {
    int tile = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = tile * kTileRows;
      const int n = (counts[e] + kTileRows - 1) / kTileRows;
      for (int j = 0; j < n; ++j) tile_expert[tile + j] = e;
      tile += n;
      counts[e] = 0;   // now the fill level
    }
  }
  __syncthreads();
  for (int i = tid; i < pairs; i += 1024) {
    const int e = ids[i];
    const int row = first[e] + atomicAdd(&counts[e], 1);
    row_pair[row] = i;
    pair_row[i] = row;
  }
}

__device__ __forceinline__ bf16x8 load8(const bf16_t* p, bool ok) {
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  return ok ? *reinterpret_cast<const bf16x8*>(p) : zero;
}

// grid (tiles, ceil(ff / 64)); block 256 = 2 x 2 waves; a wave owns 32 rows x 32 columns of gate and of up
__global__ void __launch_bounds__(256)
grouped_gate_up_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const int* __restrict__ tile_expert,
                       const int* __restrict__ row_pair, bf16_t* __restrict__ act_out, int top, int ff, int width,
                       int act) {
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, r = lane % 16, g = lane / 16;
  const int row0 = tile * kTileRows + (wave / 2) * 32;
  const int col0 = blockIdx.y * 64 + (wave % 2) * 32;
  const bf16_t* we = w + (size_t)e * 2 * ff * width;
  const bf16_t* xrow[2];
  bool xok[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int pair = row_pair[row0 + rt * 16 + r];
    xok[rt] = pair >= 0;
    xrow[rt] = x + (size_t)(pair >= 0 ? pair / top : 0) * width;
  }
  const bf16_t* grow[2];
  const bf16_t* urow[2];
  bool cok[2];
#pragma unroll
  for (int ct = 0; ct < 2; ++ct) {
    const int col = col0 + ct * 16 + r;
    cok[ct] = col < ff;
    grow[ct] = we + (size_t)(cok[ct] ? col : 0) * width;
    urow[ct] = we + (size_t)(ff + (cok[ct] ? col : 0)) * width;
  }
  f32x4 ga[2][2], ua[2][2];
#pragma unroll
  for (int ct = 0; ct < 2; ++ct)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) ga[ct][rt] = ua[ct][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < width; k0 += 32) {
    const int k = k0 + 8 * g;
    const bool kok = k < width;
    bf16x8 xb[2], gw[2], uw[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) xb[rt] = load8(xrow[rt] + k, kok && xok[rt]);
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      gw[ct] = load8(grow[ct] + k, kok && cok[ct]);
      uw[ct] = load8(urow[ct] + k, kok && cok[ct]);
    }
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        ga[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gw[ct], xb[rt], ga[ct][rt], 0, 0, 0);
        ua[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uw[ct], xb[rt], ua[ct][rt], 0, 0, 0);
      }
  }
  // lane (r, g) holds columns col0 + ct * 16 + 4g .. + 3 of row row0 + rt * 16 + r
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int row = row0 + rt * 16 + r;
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const int col = col0 + ct * 16 + 4 * g;
      if (col + 3 < ff) {
        bf16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = static_cast<__bf16>(expert_activation(ga[ct][rt][i], act) * ua[ct][rt][i]);
        *reinterpret_cast<bf16x4*>(act_out + (size_t)row * ff + col) = o;
      } else {
        for (int i = 0; i < 4; ++i)
          if (col + i < ff)
            act_out[(size_t)row * ff + col + i] = static_cast<bf16_t>(expert_activation(ga[ct][rt][i], act) * ua[ct][rt][i]);
      }
    }
  }
}

// grid (tiles, ceil(width / 128)); block 256 = 2 x 2 waves; a wave owns 32 rows x 64 columns
__global__ void __launch_bounds__(256)
grouped_down_kernel(const bf16_t* __restrict__ act_in, const bf16_t* __restrict__ w, const int* __restrict__ tile_expert,
                    float* __restrict__ y, int ff, int width) {
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, r = lane % 16, g = lane / 16;
  const int row0 = tile * kTileRows + (wave / 2) * 32;
  const int col0 = blockIdx.y * 128 + (wave % 2) * 64;
  const bf16_t* we = w + (size_t)e * width * ff;
  const bf16_t* arow[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) arow[rt] = act_in + (size_t)(row0 + rt * 16 + r) * ff;
  const bf16_t* wrow[4];
  bool cok[4];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct) {
    const int col = col0 + ct * 16 + r;
    cok[ct] = col < width;
    wrow[ct] = we + (size_t)(cok[ct] ? col : 0) * ff;
  }
  f32x4 acc[4][2];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) acc[ct][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < ff; k0 += 32) {
    const int k = k0 + 8 * g;
    const bool kok = k < ff;
    bf16x8 ab[2], wa[4];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) ab[rt] = load8(arow[rt] + k, kok);
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) wa[ct] = load8(wrow[ct] + k, kok && cok[ct]);
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) acc[ct][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[ct], ab[rt], acc[ct][rt], 0, 0, 0);
  }
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int row = row0 + rt * 16 + r;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
      const int col = col0 + ct * 16 + 4 * g;
      if (col + 3 < width) {
        *reinterpret_cast<f32x4*>(y + (size_t)row * width + col) = acc[ct][rt];
      } else {
        for (int i = 0; i < 4; ++i)
          if (col + i < width) y[(size_t)row * width + col + i] = acc[ct][rt][i];
      }
    }
  }
}

__global__ void experts_combine_kernel(const float* __restrict__ y, const int* __restrict__ pair_row,
                                       const float* __restrict__ weights, bf16_t* __restrict__ out, int top, int width) {
  const size_t t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float total = 0.f;
    for (int k = 0; k < top; ++k) total += weights[t * top + k] * y[(size_t)pair_row[t * top + k] * width + c];
    out[t * width + c] = static_cast<bf16_t>(total);
  }
}

// Rows of the padded, sorted layout for `pairs` pairs over `experts` experts (an upper bound, in whole tiles).
ATOM_EXPORT int atom_experts_grouped_tiles(int pairs, int experts) { return pairs / kTileRows + experts; }

ATOM_EXPORT int atom_experts_grouped_supports(int ff, int width, int experts) {
  return ff > 0 && width > 0 && ff % 8 == 0 && width % 8 == 0 && experts > 0 && experts <= 4096;
}

// x [tokens, width] bf16; gate_up [experts, 2 ff, width]; down [experts, width, ff]; ids, weights [tokens, top];
// scratch: tile_expert [tiles], row_pair [tiles * 64], pair_row [tokens * top] (int32), act [tiles * 64, ff] bf16
// (rows of padding are never read for a live row), y [tiles * 64, width] float32; out [tokens, width] bf16.
ATOM_EXPORT int atom_experts_grouped(const void* x, const void* gate_up, const void* down, const int* ids,
                                     const float* weights, int* tile_expert, int* row_pair, int* pair_row, void* act_buf,
                                     float* y, void* out, int tokens, int top, int experts, int ff, int width, int act,
                                     hipStream_t stream) {
  if (tokens < 0 || top <= 0 || act < 0 || act > 2) return ATOM_BAD_SHAPE;
  if (!atom_experts_grouped_supports(ff, width, experts)) return ATOM_UNSUPPORTED;
  if (tokens == 0) return ATOM_OK;
  const int pairs = tokens * top;
  const int tiles = atom_experts_grouped_tiles(pairs, experts);
  if (tiles > 0x7fffffff / kTileRows) return ATOM_TOO_LARGE;
  hipLaunchKernelGGL(experts_sort_kernel, dim3(1), dim3(1024), 2 * experts * sizeof(int), stream, ids, pairs, experts,
                     tiles, tile_expert, row_pair, pair_row);
  hipLaunchKernelGGL(grouped_gate_up_kernel, dim3(tiles, (ff + 63) / 64), dim3(256), 0, stream, (const bf16_t*)x,
                     (const bf16_t*)gate_up, tile_expert, row_pair, (bf16_t*)act_buf, top, ff, width, act);
  hipLaunchKernelGGL(grouped_down_kernel, dim3(tiles, (width + 127) / 128), dim3(256), 0, stream, (const bf16_t*)act_buf,
                     (const bf16_t*)down, tile_expert, y, ff, width);
  hipLaunchKernelGGL(experts_combine_kernel, dim3(tokens), dim3(256), 0, stream, y, pair_row, weights, (bf16_t*)out, top,
                     width);
  return launch_status();
}
