// The gated delta rule: a recurrent mixer whose state per head is a matrix S [dim, vdim] in float32.
//
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          token by token
//
// with q and k made unit vectors per head (q also times dim^-1/2), beta = sigmoid(b), and
// g = exp(-exp(A_log) softplus(a + dt_bias)), all in float32.  Before that, q, k and v pass a short causal
// convolution over time per channel and SiLU; the convolution's last taps - 1 inputs are carried per request.
//
// A request's memory is one float32 row of its state slot: [conv inputs (taps - 1) x channels | S of every head].
// Requests are walked through the step's device arrays (cu_seqlens_q, slot_of_seq), so the same kernels serve
// prompt portions, single tokens and padded rows (slot < 0: nothing is read or written) of a replayed graph.
//
//   conv_silu_state   one thread per (request, channel, run of 64 tokens); optionally a bias per channel, and SiLU or
//                     no activation
//   delta_prepare     a block per token: unit q and k, decays from their raw inputs, in place
//   delta_rule        blocks per (request, head, group of columns); a column of S (over dim) sits in the registers of up
//                     to 16 adjacent lanes, so the columns never meet; q, k and the gates of a run of tokens are
//                     staged in LDS
//   delta_out         o / rms(o) * w * silu(gate) (or sigmoid(gate)), rounded to the serving type
#include "common.h"

#include <type_traits>

constexpr int kMaxTaps = 16;

constexpr int kConvRun = 64;   // tokens of a request that one block takes

// grid (channel blocks, requests, runs of 64 tokens).  Only a request's first run reads the carried inputs, and it
// alone writes them back (after its reads), so the runs never meet.
template <typename TW>
__global__ void __launch_bounds__(256)
conv_silu_state_kernel(const float* __restrict__ x, int ldx, const TW* __restrict__ taps_w, int taps, int channels,
                       float* __restrict__ state, long slot_stride, const int* __restrict__ cu_seqlens,
                       const int* __restrict__ slot_of_seq, float* __restrict__ y, const float* __restrict__ bias,
                       int act) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int seq = blockIdx.y;
  if (c >= channels) return;
  const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
  const int first = begin + blockIdx.z * kConvRun;
  if (first >= end && !(blockIdx.z == 0)) return;
  const int last = first + kConvRun < end ? first + kConvRun : end;
  const int slot = slot_of_seq[seq];
  if (slot < 0) {
    for (int t = first; t < last; ++t) y[(size_t)t * channels + c] = 0.f;
    return;
  }
  float w[kMaxTaps], win[kMaxTaps];   // win[taps - 1] is the current input
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) {
    w[j] = j < taps ? to_f32(taps_w[(size_t)c * taps + j]) : 0.f;
    win[j] = 0.f;
  }
  const float b = bias != nullptr ? bias[c] : 0.f;
  float* tail = state + (size_t)slot * slot_stride;   // [taps - 1, channels], oldest first
  // the taps - 1 inputs before `first`: the step's own tokens where there are enough, else the carried ones
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j) {
    if (j < taps - 1) {
      const int t = first - (taps - 1) + j;   // the token whose input this is
      win[j + 1] = t >= begin ? x[(size_t)t * ldx + c] : tail[(size_t)(j + (first - begin)) * channels + c];
    }
  }
  for (int t = first; t < last; ++t) {
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j) win[j] = win[j + 1];
    const float cur = x[(size_t)t * ldx + c];
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j)
      if (j == taps - 1) win[j] = cur;
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j)
      if (j < taps) s = fmaf(w[j], win[j], s);
    s += b;
    y[(size_t)t * channels + c] = act == 0 ? s / (1.f + expf(-s)) : s;
  }
  if (blockIdx.z == 0) {
    // the request's last taps - 1 inputs after this step
    const int n = end - begin;
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j) {
      if (j < taps - 1) {
        const int back = taps - 1 - j;          // this entry is the input `back` tokens before the next one
        float v;
        if (back <= n) v = x[(size_t)(end - back) * ldx + c];
        else v = tail[(size_t)(j + n) * channels + c];   // still one of the carried ones, moved up by n
        win[j] = v;
      }
    }
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j)
      if (j < taps - 1) tail[(size_t)j * channels + c] = win[j];
  }
}

ATOM_EXPORT int atom_conv_silu_state(const float* x, int ldx, const void* taps_w, int w_dtype, int taps, int channels,
                                     float* state, long slot_stride, const int* cu_seqlens, const int* slot_of_seq,
                                     int num_seqs, int max_q_len, float* y, const float* bias, int act,
                                     hipStream_t stream) {
  if (taps < 1 || taps > kMaxTaps) return ATOM_TOO_LARGE;
  if (act != 0 && act != 1) return ATOM_UNSUPPORTED;   // 0: SiLU, 1: none
  if (channels <= 0 || ldx < channels || num_seqs < 0 || slot_stride < (long)(taps - 1) * channels) return ATOM_BAD_SHAPE;
  if (x == nullptr || taps_w == nullptr || state == nullptr || y == nullptr || max_q_len < 0) return ATOM_BAD_SHAPE;
  if (num_seqs == 0) return ATOM_OK;
  const int runs = max_q_len > 0 ? (max_q_len + kConvRun - 1) / kConvRun : 1;
  if (num_seqs > 65535 || runs > 65535) return ATOM_TOO_LARGE;
  dim3 grid((channels + 255) / 256, num_seqs, runs), block(256);
  ATOM_DISPATCH_DTYPE(w_dtype, hipLaunchKernelGGL((conv_silu_state_kernel<T>), grid, block, 0, stream, x, ldx,
                                                   (const T*)taps_w, taps, channels, state, slot_stride, cu_seqlens,
                                                   slot_of_seq, y, bias, act));
  return launch_status();
}

// ------------------------------------------------------------------ the recurrence

// The sum of v over the LPC adjacent lanes that share a column, in each of them, through the data-parallel
// permutes of one row of 16 lanes (no trip through LDS): neighbours, pairs, then the mirrored half-row and row,
// which hold the same sums as the lanes they stand for once the smaller groups are summed.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

template <int LPC>
__device__ __forceinline__ float group_sum(float v) {
  if constexpr (LPC >= 2) v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  if constexpr (LPC >= 4) v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  if constexpr (LPC >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
  if constexpr (LPC >= 16) v = dpp_add<0x140>(v);  // row_mirror
  return v;
}

// What does not depend on the state is done for all tokens side by side, in place, before the recurrence walks them:
// q and k become unit vectors per head (q also times dim^-1/2), and the raw decay inputs become the decays
// exp(-exp(A_log) softplus(a + dt_bias)), one per head or one per head and key channel.  A block per token.
__global__ void __launch_bounds__(256)
delta_prepare_kernel(float* __restrict__ qkv, int channels, float* __restrict__ dec, int ld_dec, int a_off,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias, int heads, int kv_heads, int dim,
                     int per_head) {
  const size_t t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const float q_scale = 1.f / sqrtf((float)dim);
  for (int row = wave; row < 2 * kv_heads; row += 256 / kWave) {
    float* r = qkv + t * channels + (size_t)row * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += kWave) ss += r[i] * r[i];
    ss = wave_sum(ss);
    const float f = (row < kv_heads ? q_scale : 1.f) / sqrtf(ss + 1e-6f);
    for (int i = lane; i < dim; i += kWave) r[i] *= f;
  }
  float* d = dec + t * ld_dec + a_off;
  const int wide = heads * per_head;
  for (int i = threadIdx.x; i < wide; i += blockDim.x) {
    const float z = d[i] + dt_bias[i];
    const float sp_z = z > 20.f ? z : log1pf(expf(z));
    d[i] = expf(-expf(a_log[i / per_head]) * sp_z);
  }
}

constexpr int kRun = 16;   // tokens whose q, k and gates are staged at once
constexpr int kDPL = 16;   // entries of a column of S that one lane holds (8 for heads of 65 to 128 key channels, whose
                           // columns then spread over 16 lanes: half the multiply-adds a token and wave, twice the waves)

// qkv [T, channels] float32 after convolution and SiLU: q heads (kv_heads x dim) | k heads | v heads (heads x vdim).
// ab [T, ld_ab] float32: the raw decay inputs at a_off and the raw beta inputs at b_off, one per head.
// A column of S (dim entries) is spread over LPC adjacent lanes, entries 16 s .. 16 s + 15 in lane s of them (a lane's
// part of a staged q, k or decay row is then 64 consecutive bytes of LDS, read 16 bytes at a time), so that a token costs
// each lane 16 entries and two sums over the LPC lanes; the sums over a lane's entries run in four independent chains.
//
// CHANNEL: the decay is one number per head and key channel (row of S): dec holds heads x dim raw inputs a token at
// a_off, dt_bias heads x dim entries, and a run's decays are staged like its q and k rows.
template <int LPC, bool CHANNEL, int DPL = kDPL>
__global__ void __launch_bounds__(256)
delta_rule_kernel(const float* __restrict__ qkv, int channels, const float* __restrict__ ab, int ld_ab,
                  const float* __restrict__ dec, int ld_dec, int a_off,
                  int b_off,
                  float* __restrict__ state, long slot_stride, long state_off, const int* __restrict__ cu_seqlens,
                  const int* __restrict__ slot_of_seq, float* __restrict__ out, int heads, int kv_heads, int dim,
                  int vdim) {
  constexpr int DMAX = DPL * LPC;
  __shared__ __attribute__((aligned(16))) float qs[kRun][DMAX];
  __shared__ __attribute__((aligned(16))) float ks[kRun][DMAX];
  __shared__ __attribute__((aligned(16))) float gv[CHANNEL ? kRun : 1][DMAX];   // CHANNEL: a run's decays per key channel
  __shared__ float gs[kRun], bs[kRun];
  const int head = blockIdx.x, seq = blockIdx.y;
  const int tid = threadIdx.x;
  const int sub = tid % LPC;
  const int col = blockIdx.z * (256 / LPC) + tid / LPC;   // this lane's column of S
  const int kvh = head / (heads / kv_heads);
  const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
  const int slot = slot_of_seq[seq];
  const bool live = col < vdim;
  if (slot < 0) {
    for (int t = begin; t < end; ++t)
      if (live && sub == 0) out[((size_t)t * heads + head) * vdim + col] = 0.f;
    return;
  }
  float* sp = state + (size_t)slot * slot_stride + state_off + (size_t)head * dim * vdim;   // [dim, vdim]
  float S[DPL];
#pragma unroll
  for (int j = 0; j < DPL; ++j) {
    const int i = sub * DPL + j;
    S[j] = (live && i < dim) ? sp[(size_t)i * vdim + col] : 0.f;
  }
  const int k_off = kv_heads * dim, v_off = 2 * kv_heads * dim;
  // A run's q and k rows, its values of this column and its gates travel memory -> registers -> LDS; the registers
  // are filled for the next run while this run's tokens are worked through, so that no load is waited for inside
  // the chain of tokens.
  constexpr int QK_ITEMS = 2 * kRun * DMAX / 256;
  constexpr int G_ITEMS = CHANNEL ? kRun * DMAX / 256 : 1;
  float qk_raw[QK_ITEMS], g_raw[G_ITEMS], v_next[kRun], a_next = 0.f, b_next = 0.f;
  auto load_run = [&](int t0) {
    const int n = end - t0 < kRun ? end - t0 : kRun;
#pragma unroll
    for (int it = 0; it < QK_ITEMS; ++it) {
      const int idx = tid + it * 256;
      const int item = idx / DMAX, i = idx % DMAX;
      const int j = item >> 1, is_k = item & 1;
      qk_raw[it] = (j < n && i < dim) ? qkv[(size_t)(t0 + j) * channels + (is_k ? k_off : 0) + kvh * dim + i] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < kRun; ++j)
      v_next[j] = (live && j < n) ? qkv[(size_t)(t0 + j) * channels + v_off + head * vdim + col] : 0.f;
    if constexpr (CHANNEL) {
#pragma unroll
      for (int it = 0; it < G_ITEMS; ++it) {
        const int idx = tid + it * 256;
        const int j = idx / DMAX, i = idx % DMAX;
        g_raw[it] = (j < n && i < dim) ? dec[(size_t)(t0 + j) * ld_dec + a_off + head * dim + i] : 0.f;
      }
    }
    if (tid < n) {
      const float* r = ab + (size_t)(t0 + tid) * ld_ab;
      if constexpr (!CHANNEL) a_next = dec[(size_t)(t0 + tid) * ld_dec + a_off + head];
      b_next = r[b_off + head];
    }
  };
  if (begin < end) load_run(begin);
  for (int t0 = begin; t0 < end; t0 += kRun) {
    const int n = end - t0 < kRun ? end - t0 : kRun;
    __syncthreads();   // the previous run's q and k have been read
#pragma unroll
    for (int it = 0; it < QK_ITEMS; ++it) {
      const int idx = tid + it * 256;
      const int item = idx / DMAX, i = idx % DMAX;
      ((item & 1) ? ks[item >> 1] : qs[item >> 1])[i] = qk_raw[it];
    }
    if constexpr (CHANNEL) {
#pragma unroll
      for (int it = 0; it < G_ITEMS; ++it) {
        const int idx = tid + it * 256;
        const int j = idx / DMAX, i = idx % DMAX;
        gv[j][i] = g_raw[it];
      }
    }
    if (tid < n) {
      if constexpr (!CHANNEL) gs[tid] = a_next;
      bs[tid] = 1.f / (1.f + expf(-b_next));
    }
    float vv[kRun];
#pragma unroll
    for (int j = 0; j < kRun; ++j) vv[j] = v_next[j];
    __syncthreads();
    if (t0 + kRun < end) load_run(t0 + kRun);
    // a token's k and q entries are read from LDS one token ahead of their use, so that the chain below never
    // waits for them
    float kc[DPL], qc[DPL], kn[DPL], qn[DPL];
    float gc[CHANNEL ? DPL : 1], gn[CHANNEL ? DPL : 1];
#pragma unroll
    for (int e = 0; e < DPL; ++e) {
      kc[e] = ks[0][sub * DPL + e];
      qc[e] = qs[0][sub * DPL + e];
      if constexpr (CHANNEL) gc[e] = gv[0][sub * DPL + e];
    }
    // A whole run is walked without a test per token: the registers that hold the next token's entries then simply
    // become the current ones, with no copies (a test per token makes every hand-over a set of moves).
    auto walk = [&](auto whole) {
#pragma unroll
    for (int j = 0; j < kRun; ++j) {
      if (decltype(whole)::value || j < n) {
      const float g = CHANNEL ? 1.f : gs[j];
      const float beta = bs[j];
      const float v = vv[j];

      if (j + 1 < kRun) {
#pragma unroll
        for (int e = 0; e < DPL; ++e) {
          kn[e] = ks[j + 1][sub * DPL + e];
          qn[e] = qs[j + 1][sub * DPL + e];
          if constexpr (CHANNEL) gn[e] = gv[j + 1][sub * DPL + e];
        }
      }
      float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < DPL; ++e) {
        if constexpr (CHANNEL) S[e] *= gc[e]; else S[e] *= g;
        part[e & 3] = fmaf(S[e], kc[e], part[e & 3]);
      }
      const float dot = group_sum<LPC>((part[0] + part[1]) + (part[2] + part[3]));
      const float u = beta * (v - dot);
      part[0] = part[1] = part[2] = part[3] = 0.f;
#pragma unroll
      for (int e = 0; e < DPL; ++e) {
        S[e] = fmaf(kc[e], u, S[e]);
        part[e & 3] = fmaf(S[e], qc[e], part[e & 3]);
      }
      const float o = group_sum<LPC>((part[0] + part[1]) + (part[2] + part[3]));
      if (live && sub == 0) out[((size_t)(t0 + j) * heads + head) * vdim + col] = o;
#pragma unroll
      for (int e = 0; e < DPL; ++e) {
        kc[e] = kn[e];
        qc[e] = qn[e];
        if constexpr (CHANNEL) gc[e] = gn[e];
      }
      }
    }
    };
    if (n == kRun) walk(std::true_type{});
    else walk(std::false_type{});
  }
#pragma unroll
  for (int j = 0; j < DPL; ++j) {
    const int i = sub * DPL + j;
    if (live && i < dim) sp[(size_t)i * vdim + col] = S[j];
  }
}

// qkv and the decay inputs are changed in place (see delta_prepare_kernel); tokens is the number of their rows.
ATOM_EXPORT int atom_delta_rule(float* qkv, int tokens, int channels, const float* ab, int ld_ab, float* dec, int ld_dec,
                                int a_off, int b_off, int per_channel,
                                const float* a_log, const float* dt_bias, float* state, long slot_stride,
                                long state_off, const int* cu_seqlens, const int* slot_of_seq, int num_seqs, float* out,
                                int heads, int kv_heads, int dim, int vdim, hipStream_t stream) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0 || num_seqs < 0) return ATOM_BAD_SHAPE;
  if (channels != 2 * kv_heads * dim + heads * vdim) return ATOM_BAD_SHAPE;
  if (a_off < 0 || b_off < 0 || b_off + heads > ld_ab) return ATOM_BAD_SHAPE;
  if (a_off + heads * (per_channel ? dim : 1) > ld_dec) return ATOM_BAD_SHAPE;
  if (ab == nullptr || dec == nullptr) return ATOM_BAD_SHAPE;
  if (state_off < 0 || slot_stride < state_off + (long)heads * dim * vdim) return ATOM_BAD_SHAPE;
  if (dim > 256) return ATOM_TOO_LARGE;
  if (num_seqs == 0 || tokens <= 0) return ATOM_OK;
  if (num_seqs > 65535 || heads > 65535) return ATOM_TOO_LARGE;
  hipLaunchKernelGGL(delta_prepare_kernel, dim3(tokens), dim3(256), 0, stream, qkv, channels, dec, ld_dec, a_off, a_log,
                     dt_bias, heads, kv_heads, dim, per_channel ? dim : 1);
  int lpc = 1;
  while (lpc * kDPL < dim) lpc *= 2;
  const bool narrow = dim > 64 && dim <= 128;   // 16 lanes of 8 entries instead of 8 lanes of 16
  if (narrow) lpc = 16;
  const int cols = 256 / lpc;
  dim3 grid(heads, num_seqs, (vdim + cols - 1) / cols), block(256);
  if (grid.z > 65535) return ATOM_TOO_LARGE;
#define LAUNCH_AS(L, C)                                                                                          \
  hipLaunchKernelGGL((delta_rule_kernel<L, C>), grid, block, 0, stream, qkv, channels, ab, ld_ab, dec, ld_dec, a_off, \
                     b_off, state, slot_stride, state_off, cu_seqlens, slot_of_seq, out, heads, kv_heads, dim, vdim)
#define LAUNCH(L)                  \
  do {                             \
    if (per_channel) {             \
      LAUNCH_AS(L, true);          \
    } else {                       \
      LAUNCH_AS(L, false);         \
    }                              \
  } while (0)
  if (narrow) {
    if (per_channel)
      hipLaunchKernelGGL((delta_rule_kernel<16, true, 8>), grid, block, 0, stream, qkv, channels, ab, ld_ab, dec, ld_dec,
                         a_off, b_off, state, slot_stride, state_off, cu_seqlens, slot_of_seq, out, heads, kv_heads, dim,
                         vdim);
    else
      hipLaunchKernelGGL((delta_rule_kernel<16, false, 8>), grid, block, 0, stream, qkv, channels, ab, ld_ab, dec, ld_dec,
                         a_off, b_off, state, slot_stride, state_off, cu_seqlens, slot_of_seq, out, heads, kv_heads, dim,
                         vdim);
    return launch_status();
  }
  switch (lpc) {
    case 1: LAUNCH(1); break;
    case 2: LAUNCH(2); break;
    case 4: LAUNCH(4); break;
    case 8: LAUNCH(8); break;
    default: LAUNCH(16); break;
  }
#undef LAUNCH
#undef LAUNCH_AS
  return launch_status();
}

// ------------------------------------------------------------------ the read-out's norm and gate
//
// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * w * silu(gate[t, h, :]);  a wave per (token, head)

template <typename T>
__global__ void __launch_bounds__(256)
delta_out_kernel(const float* __restrict__ o, const float* __restrict__ gate, int ld_gate, int gate_off,
                 const float* __restrict__ w, float eps, T* __restrict__ y, int heads, int vdim, size_t items,
                 int act) {
  const size_t item = (size_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (item >= items) return;
  const int lane = threadIdx.x % kWave;
  const size_t t = item / heads;
  const int h = (int)(item - t * heads);
  const float* src = o + item * vdim;
  const float* gr = gate + t * ld_gate + gate_off + (size_t)h * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += kWave) ss += src[i] * src[i];
  const float rstd = 1.f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  T* dst = y + item * vdim;
  for (int i = lane; i < vdim; i += kWave) {
    const float g = gr[i];
    const float sig = 1.f / (1.f + expf(-g));
    dst[i] = from_f32<T>(src[i] * rstd * w[i] * (act == 0 ? g * sig : sig));
  }
}

ATOM_EXPORT int atom_delta_out(const float* o, const float* gate, int ld_gate, int gate_off, const float* w, float eps,
                               void* y, int dtype, int tokens, int heads, int vdim, int act, hipStream_t stream) {
  if (act != 0 && act != 1) return ATOM_UNSUPPORTED;   // 0: SiLU of the gate, 1: its sigmoid
  if (tokens < 0 || heads <= 0 || vdim <= 0 || gate_off < 0 || gate_off + heads * vdim > ld_gate) return ATOM_BAD_SHAPE;
  if (o == nullptr || gate == nullptr || w == nullptr || y == nullptr) return ATOM_BAD_SHAPE;
  const size_t items = (size_t)tokens * heads;
  if (items == 0) return ATOM_OK;
  const size_t blocks = (items + 3) / 4;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((delta_out_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, o,
                                                 gate, ld_gate, gate_off, w, eps, (T*)y, heads, vdim, items, act));
  return launch_status();
}
