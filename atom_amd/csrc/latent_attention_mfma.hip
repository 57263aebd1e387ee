// Attention over the latent pages on the matrix cores (bfloat16 in, float32 accumulate), gfx950.
//
// All heads of a token read the same cached rows [rank | rot], as keys (all of a row) and as values (its first
// `rank` entries).  A block of four waves owns up to 64 rows (token, head) of one request (`tpt` consecutive
// tokens times `hpt` heads) and one range of keys; it walks the range 32 keys at a time.  A chunk is read from its
// pages once and staged in LDS twice: row-major [key][width] for the scores and transposed [entry][key] for the
// weighted sum, since no transposed copy of the cache exists.  Both products are formed transposed, so that a lane
// always holds values of ONE row (row = lane % 16):
//
//     S^T[key][row] = K[key][:] . Q[row][:]           A = K rows from LDS, B = Q (registers)
//     O^T[e][row]   = V^T[e][key] . P[row][key]       A = V^T rows from LDS, B = P
//
// The two score tiles of a chunk take their 16 keys each in the order that leaves lane (row, g = lane / 16) with
// the scores of keys 8g .. 8g + 7, which is the B operand of one v_mfma_f32_16x16x32_bf16 of the second product.
// A row's running maximum, sum and rescale factor are per-lane scalars.  Softmax is float32; the sink joins the
// denominator at the end.
//
// Prompt portions: every block takes all keys of its tile.  Single tokens: a row's keys are split over `parts`
// blocks (whole chunks each), whose unnormalised results and (maximum, sum) a second kernel merges.
// Causal by absolute position; optional window.  Needs width % 8 == 0 and rank % 16 == 0.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

struct LatentParams {
  const bf16_t* q;          // [tokens, heads, width], scaled
  const bf16_t* pages;      // [num_pages * page_size, width]
  bf16_t* out;              // [tokens, heads, rank]
  float* ws_o;              // parts > 1: [tokens, heads, parts, rank]
  float* ws_ml;             // parts > 1: [tokens, heads, parts, 2]
  const int* cu_q;          // [num_seqs + 1]
  const int* ctx_lens;      // [num_seqs]
  const int* block_tables;  // [num_seqs, max_blocks]
  const float* sink;        // [heads] or null
  int num_seqs, max_blocks, heads, rank, width, page_size, window, parts, hpt, tpt;
  int page_shift;           // log2(page_size) where that is a power of two of at least 8, else -1
};

constexpr int kLChunk = 32;
constexpr int kVPitch = kLChunk * 2 + 16;   // bytes of a transposed row: 32 keys and a pad that spreads the banks

__host__ __device__ inline int latent_k_pitch(int width) {
  const int steps = (width + 31) / 32;
  return (steps * 64 + 127) / 128 * 128 + 16;
}

template <int RT, int KS>
__global__ void __launch_bounds__(256) latent_mfma_kernel(LatentParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x;
  const int kpitch = latent_k_pitch(p.width);
  unsigned char* klds = lds;
  unsigned char* vlds = lds + kLChunk * kpitch;
  const int steps = (p.width + 31) / 32;

  // which request and which of its tokens: tiles are numbered request by request
  int b = blockIdx.x, seq = -1, q_len = 0, q_start = 0;
  for (int s = 0; s < p.num_seqs; ++s) {
    const int ql = p.cu_q[s + 1] - p.cu_q[s];
    const int n = (ql + p.tpt - 1) / p.tpt;
    if (b < n) {
      seq = s;
      q_len = ql;
      q_start = p.cu_q[s];
      break;
    }
    b -= n;
  }
  if (seq < 0) return;
  const int t0 = b * p.tpt;
  const int ctx = p.ctx_lens[seq];
  const int cached = ctx - q_len;
  const int tokens_here = (q_len - t0 < p.tpt) ? q_len - t0 : p.tpt;
  const int h0 = blockIdx.y * p.hpt;
  const int last_pos = cached + t0 + tokens_here - 1;
  const int* table = p.block_tables + (size_t)seq * p.max_blocks;

  const int wave = tid / kWave, lane = tid % kWave, r = lane % 16, g = lane / 16;
  const int R = wave * 16 + r;
  const int tt = R / p.hpt;
  const int head = h0 + R % p.hpt;
  const bool row_ok = ctx > 0 && cached >= 0 && tt < tokens_here && tt < p.tpt && head < p.heads;
  const int token = q_start + t0 + tt;
  const int pos_r = cached + t0 + tt;
  const int lo_r = (p.window > 0 && pos_r - p.window + 1 > 0) ? pos_r - p.window + 1 : 0;
  const bool wave_busy = __ballot(row_ok) != 0;

  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int k0 = ks * 32 + g * 8;
    qreg[ks] = (row_ok && k0 < p.width)
                   ? *reinterpret_cast<const bf16x8*>(p.q + ((size_t)token * p.heads + head) * p.width + k0)
                   : zero8;
  }
  // the columns between width and the next multiple of 32 stay zero for the whole kernel
  {
    const int padded = steps * 32;
    const int extra = padded - p.width;
    for (int item = tid; item < kLChunk * extra; item += 256) {
      const int j = item / extra, cidx = p.width + item % extra;
      *reinterpret_cast<bf16_t*>(klds + j * kpitch + cidx * 2) = static_cast<bf16_t>(0.f);
    }
  }

  f32x4 acc[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  // the chunks of this block
  int my_lo = 0, my_hi = 0;
  if (ctx > 0 && cached >= 0 && last_pos >= 0) {
    const int first_key = (p.window > 0 && cached + t0 - p.window + 1 > 0) ? cached + t0 - p.window + 1 : 0;
    const int c_lo = first_key / kLChunk, c_hi = last_pos / kLChunk + 1;
    const int per = (c_hi - c_lo + p.parts - 1) / p.parts;
    my_lo = c_lo + (int)blockIdx.z * per;
    my_hi = my_lo + per < c_hi ? my_lo + per : c_hi;
  }
  const int groups = p.width / 8;
  const int keyA0 = 8 * (r / 4) + (r % 4);   // the key of A row r in the first score tile; the second: + 4

  // a chunk's rows travel memory -> registers -> LDS; the registers are filled for the next chunk while this one
  // is multiplied, so that the memory's latency is hidden behind the products.  Work is dealt out with the pair of
  // keys running fastest: 16 lanes then write 16 consecutive words of a transposed row (consecutive banks), and
  // four such groups of lanes read one whole 64-byte line of each of their 32 rows.
  constexpr int ITEMS = (KS * 64 + 255) / 256;   // (pair of keys, 8 entries) items a thread moves, at most
  bf16x8 ra[ITEMS], rb[ITEMS];
  // without a branch: every lookup and every row load of a chunk is asked for before any is waited for.  Keys
  // beyond the last visible one are read as that one and replaced by zeros when they are staged.
  const int n_items = (kLChunk / 2) * groups;
  auto fetch = [&](int c) {
    const int kbase = c * kLChunk;
    size_t row_a[ITEMS], row_b[ITEMS];
    if (p.page_shift >= 0) {
      // pages of 8, 16, 32, ... keys: a chunk lies in at most four pages, whose numbers every lane needs alike
      // (uniform loads), and places within a page are shifts and masks
      const int pbase = kbase >> p.page_shift, plast = last_pos >> p.page_shift;
      int tab[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) tab[j] = table[pbase + j < plast ? pbase + j : plast];
      const int mask = p.page_size - 1;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int item = tid + it * 256 < n_items ? tid + it * 256 : n_items - 1;
        const int kp = item % (kLChunk / 2);
        const int key0 = kbase + 2 * kp < last_pos ? kbase + 2 * kp : last_pos;
        const int key1 = key0 + 1 < last_pos ? key0 + 1 : last_pos;
        const int j0 = (key0 >> p.page_shift) - pbase, j1 = (key1 >> p.page_shift) - pbase;
        const int page0 = j0 == 0 ? tab[0] : j0 == 1 ? tab[1] : j0 == 2 ? tab[2] : tab[3];
        const int page1 = j1 == 0 ? tab[0] : j1 == 1 ? tab[1] : j1 == 2 ? tab[2] : tab[3];
        row_a[it] = ((size_t)page0 << p.page_shift) | (size_t)(key0 & mask);
        row_b[it] = ((size_t)page1 << p.page_shift) | (size_t)(key1 & mask);
      }
    } else {
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        const int item = tid + it * 256 < n_items ? tid + it * 256 : n_items - 1;
        const int kp = item % (kLChunk / 2);
        const int key0 = kbase + 2 * kp < last_pos ? kbase + 2 * kp : last_pos;
        const int key1 = key0 + 1 < last_pos ? key0 + 1 : last_pos;
        row_a[it] = (size_t)table[key0 / p.page_size] * p.page_size + key0 % p.page_size;
        row_b[it] = (size_t)table[key1 / p.page_size] * p.page_size + key1 % p.page_size;
      }
    }
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * 256 < n_items ? tid + it * 256 : n_items - 1;
      const int dg = item / (kLChunk / 2);
      ra[it] = *reinterpret_cast<const bf16x8*>(p.pages + row_a[it] * p.width + dg * 8);
      rb[it] = *reinterpret_cast<const bf16x8*>(p.pages + row_b[it] * p.width + dg * 8);
    }
  };
  auto stash = [&](int c) {
    const int kbase = c * kLChunk;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * 256;
      if (item < n_items) {
        const int kp = item % (kLChunk / 2), dg = item / (kLChunk / 2);
        const bf16x8 va = kbase + 2 * kp <= last_pos ? ra[it] : zero8;
        const bf16x8 vb = kbase + 2 * kp + 1 <= last_pos ? rb[it] : zero8;
        *reinterpret_cast<bf16x8*>(klds + (2 * kp) * kpitch + dg * 16) = va;
        *reinterpret_cast<bf16x8*>(klds + (2 * kp + 1) * kpitch + dg * 16) = vb;
        if (dg * 8 < p.rank) {
          // entry i of both keys side by side: the halves of the rows' 32-bit words
          const u32x4 wa = __builtin_bit_cast(u32x4, va), wb = __builtin_bit_cast(u32x4, vb);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const unsigned lo16 = (i & 1) ? wa[i / 2] >> 16 : wa[i / 2] & 0xffffu;
            const unsigned hi16 = (i & 1) ? wb[i / 2] >> 16 : wb[i / 2] & 0xffffu;
            *reinterpret_cast<unsigned*>(vlds + (dg * 8 + i) * kVPitch + kp * 4) = lo16 | (hi16 << 16);
          }
        }
      }
    }
  };
  if (my_lo < my_hi) fetch(my_lo);

  for (int c = my_lo; c < my_hi; ++c) {
    const int kbase = c * kLChunk;
    __syncthreads();   // the chunk before has been read
    stash(c);
    __syncthreads();
    // not inside a branch: the compiler waits for loads that a branch issued where the branch ends.  Past the last
    // chunk the last one is read again and never staged.
    fetch(c + 1 < my_hi ? c + 1 : my_hi - 1);
    if (!wave_busy) continue;

    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks < steps) {
        const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(klds + keyA0 * kpitch + (ks * 32 + g * 8) * 2);
        const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(klds + (keyA0 + 4) * kpitch + (ks * 32 + g * 8) * 2);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qreg[ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qreg[ks], s1, 0, 0, 0);
      }
    }
    float sc[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = kbase + 8 * g + i;
      const bool seen = row_ok && key <= pos_r && key >= lo_r;
      sc[i] = seen ? sc[i] : -INFINITY;
      mx = fmaxf(mx, sc[i]);
    }
    mx = rows_max(mx);
    const float m_new = fmaxf(m_run, mx);
    float pr[8];
    float sum = 0.f;
    float alpha = 1.f;
    if (m_new == -INFINITY) {
#pragma unroll
      for (int i = 0; i < 8; ++i) pr[i] = 0.f;
    } else {
      alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        pr[i] = (sc[i] == -INFINITY) ? 0.f : __expf(sc[i] - m_new);
        sum += pr[i];
      }
      m_run = m_new;
    }
    sum = rows_sum(sum);
    l_run = l_run * alpha + sum;
    bf16x8 pb;
#pragma unroll
    for (int i = 0; i < 8; ++i) pb[i] = static_cast<__bf16>(pr[i]);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      if (t * 16 < p.rank) {
        const bf16x8 vt = *reinterpret_cast<const bf16x8*>(vlds + (t * 16 + r) * kVPitch + g * 16);
        acc[t] *= alpha;
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pb, acc[t], 0, 0, 0);
      }
    }
  }

  if (!(tt < tokens_here && tt < p.tpt && head < p.heads)) return;
  const size_t row_index = (size_t)token * p.heads + head;
  if (p.parts == 1) {
    float denom = l_run, f = 1.f;
    if (p.sink) {
      const float sk = p.sink[head];
      const float top = fmaxf(m_run, sk);
      f = (m_run == -INFINITY) ? 0.f : __expf(m_run - top);
      denom = l_run * f + __expf(sk - top);
    }
    const float inv = denom > 0.f ? f / denom : 0.f;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int e = t * 16 + 4 * g;
      if (e < p.rank) {
        bf16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = static_cast<__bf16>(acc[t][i] * inv);
        *reinterpret_cast<bf16x4*>(p.out + row_index * p.rank + e) = o;
      }
    }
  } else {
    float* wo = p.ws_o + (row_index * p.parts + blockIdx.z) * p.rank;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int e = t * 16 + 4 * g;
      if (e < p.rank) *reinterpret_cast<f32x4*>(wo + e) = acc[t];
    }
    if (g == 0) {
      float* ml = p.ws_ml + (row_index * p.parts + blockIdx.z) * 2;
      ml[0] = m_run;
      ml[1] = l_run;
    }
  }
}

// out[row] = sum_p o_p exp(m_p - M) / (sum_p l_p exp(m_p - M) + exp(sink - M)), M the largest of the m_p and the sink
__global__ void __launch_bounds__(128)
latent_merge_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml, const float* __restrict__ sink,
                    bf16_t* __restrict__ out, int heads, int rank, int parts) {
  __shared__ float share[64];   // the parts' weights exp(m_p - M) / denominator
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const int head = (int)(row % heads);
  const int tid = threadIdx.x;
  const float* ml = ws_ml + row * parts * 2;
  const float sk = sink ? sink[head] : -INFINITY;
  const float mine = tid < parts ? ml[2 * tid] : -INFINITY;
  const float top = fmaxf(block_max(mine, scratch), sk);
  const float w = (tid < parts && mine != -INFINITY) ? __expf(mine - top) : 0.f;
  float denom = block_sum(tid < parts ? w * ml[2 * tid + 1] : 0.f, scratch);
  if (sink && top != -INFINITY) denom += __expf(sk - top);
  if (tid < parts) share[tid] = denom > 0.f ? w / denom : 0.f;
  __syncthreads();
  for (int e = tid; e < rank; e += 128) {
    float a = 0.f;
    for (int q = 0; q < parts; ++q) a += ws_o[(row * parts + q) * rank + e] * share[q];
    out[row * rank + e] = static_cast<bf16_t>(a);
  }
}

// The register sets the kernel is built for: (rank up to 16 RT, width up to 32 KS).
static int latent_variant(int rank, int width) {
  if (rank % 16 || width % 8 || rank <= 0 || width < rank) return -1;
  if (rank <= 128 && width <= 192) return 0;
  if (rank <= 256 && width <= 320) return 1;
  if (rank <= 512 && width <= 576) return 2;
  return -1;
}

ATOM_EXPORT int atom_latent_mfma_supports(int rank, int width) { return latent_variant(rank, width) >= 0; }

// Rows a block takes: heads per tile and tokens per tile for `heads` heads.
ATOM_EXPORT int atom_latent_mfma_tokens_per_tile(int heads) {
  const int hpt = heads < 64 ? heads : 64;
  return 64 / hpt;
}

ATOM_EXPORT int atom_latent_attention_mfma(const void* q, const void* pages, void* out, float* ws_o, float* ws_ml,
                                           const int* cu_q, const int* ctx_lens, const int* block_tables,
                                           int max_blocks, const float* sink, int num_seqs, int tokens, int heads,
                                           int rank, int width, int page_size, int window, int parts,
                                           hipStream_t stream) {
  if (num_seqs < 0 || tokens < 0 || heads <= 0 || page_size <= 0 || max_blocks <= 0 || parts < 1) return ATOM_BAD_SHAPE;
  const int variant = latent_variant(rank, width);
  if (variant < 0) return ATOM_UNSUPPORTED;
  if (parts > 1 && (ws_o == nullptr || ws_ml == nullptr)) return ATOM_BAD_SHAPE;
  if (tokens == 0 || num_seqs == 0) return ATOM_OK;
  LatentParams p;
  p.q = (const bf16_t*)q;
  p.pages = (const bf16_t*)pages;
  p.out = (bf16_t*)out;
  p.ws_o = ws_o;
  p.ws_ml = ws_ml;
  p.cu_q = cu_q;
  p.ctx_lens = ctx_lens;
  p.block_tables = block_tables;
  p.sink = sink;
  p.num_seqs = num_seqs;
  p.max_blocks = max_blocks;
  p.heads = heads;
  p.rank = rank;
  p.width = width;
  p.page_size = page_size;
  p.window = window;
  p.parts = parts;
  p.hpt = heads < 64 ? heads : 64;
  p.tpt = 64 / p.hpt;
  p.page_shift = -1;
  for (int sh = 3; sh < 20; ++sh)
    if (page_size == (1 << sh)) p.page_shift = sh;
  const int tiles = tokens / p.tpt + num_seqs;   // at least sum over requests of ceil(q_len / tpt)
  const int chunks = (heads + p.hpt - 1) / p.hpt;
  if (chunks > 65535 || parts > 64) return ATOM_TOO_LARGE;   // the merge holds a weight per part in LDS
  const size_t smem = (size_t)kLChunk * latent_k_pitch(width) + (size_t)rank * kVPitch;
  if (smem > 160 * 1024) return ATOM_TOO_LARGE;
  dim3 grid(tiles, chunks, parts), block(256);
#define LAUNCH(RT, KS)                                                                                             \
  do {                                                                                                             \
    static size_t allowed = 0;                                                                                     \
    if (smem > 48 * 1024 && smem > allowed) {                                                                      \
      if (hipFuncSetAttribute((const void*)latent_mfma_kernel<RT, KS>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)smem) != hipSuccess)                                                            \
        return ATOM_LAUNCH_FAILED;                                                                                 \
      allowed = smem;                                                                                              \
    }                                                                                                              \
    hipLaunchKernelGGL((latent_mfma_kernel<RT, KS>), grid, block, smem, stream, p);                                \
  } while (0)
  if (variant == 0) LAUNCH(8, 6);
  else if (variant == 1) LAUNCH(16, 10);
  else LAUNCH(32, 18);
#undef LAUNCH
  if (hipGetLastError() != hipSuccess) return ATOM_LAUNCH_FAILED;
  if (parts > 1) {
    hipLaunchKernelGGL(latent_merge_kernel, dim3(tokens * heads), dim3(128), 0, stream, ws_o, ws_ml, sink,
                       (bf16_t*)out, heads, rank, parts);
  }
  return launch_status();
}
