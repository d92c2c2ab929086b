// Attention over cached latents on the matrix cores (v_mfma_f32_16x16x32_bf16), bfloat16 in, float softmax.
//
// All query heads read the same keys [c_j ; kr_j] and the same values c_j, so a *column* is a (token, head) pair
// and a wave owns 16 consecutive columns of one request (head running fastest): every key it loads serves 16
// heads, or several tokens' heads.  The waves of a block share one tile of 16 columns and take its key blocks in turn,
// each with its own running maximum, sum and accumulators, merged through LDS at the end in wave order: a single
// decoded token's keys are then walked by four waves at once.  Keys are walked in blocks of 32:
//
//   S^T[key, col]  = K[key, :] . Q^T[:, col]      A operand: 16 keys x 32 entries read in place from the pages (the
//                                                 latent's C entries, then the rotated part's R), B: the query
//   online softmax per column in float (log2 units); a column's own position and window mask its keys; the
//   sink joins the denominator at the end
//   O^T[i, col] += c^T[i, key] . P^T[key, col]    A operand: the latent pages' transposed copy [page][C][slot],
//                                                 B: P^T straight from the S^T accumulators
//
// The sums of the exponentials come from one more product with ones (the bfloat16 values that weigh the latents).
// Values past the last visible key are zeroed before use and pages past the context are never dereferenced.
// Launch: grid (column tiles of the longest portion, requests); a block without a tile leaves at once, so the launch
// depends on the step's number of requests and longest portion only.
#include "common.h"
#include "api.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int LM_WAVES = 4;

template <int C, int R>
__global__ void __launch_bounds__(LM_WAVES * MS_WAVE)
latent_attention_mfma_kernel(const bf16* __restrict__ q, size_t q_tok, size_t q_head, const bf16* __restrict__ c_pages,
                             const bf16* __restrict__ r_pages, const bf16* __restrict__ ct_pages,
                             const int* __restrict__ block_table, int table_stride, const int* __restrict__ table_rows,
                             const int* __restrict__ q_start, const int* __restrict__ context_lens,
                             const float* __restrict__ sink, bf16* __restrict__ out, size_t out_tok, size_t out_head,
                             int H, int page_size, float scale_log2e, int window) {
  constexpr int KS_C = C / 32, KS_R = R / 32, CT = C / 16;
  __shared__ float sm_m[LM_WAVES][16], sm_l[LM_WAVES][16];
  __shared__ f32x4 sm_o[CT][MS_WAVE];
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);
  const int col16 = lane & 15, kq = lane >> 4;
  const int r = blockIdx.y;
  const int q0 = q_start[r];
  const int qlen = q_start[r + 1] - q0;
  const int ncols = qlen * H;
  const int c0 = blockIdx.x * 16;
  if (c0 >= ncols) return;                         // the whole block
  const int start_pos = context_lens[r] - qlen;
  const int* table = block_table + (size_t)(table_rows ? table_rows[r] : r) * table_stride;

  const int last_col = min(ncols, c0 + 16) - 1;
  const int key_hi = start_pos + last_col / H;
  const int key_lo = window > 0 ? max(0, start_pos + c0 / H - window + 1) : 0;

  // this lane's column
  const int c = c0 + col16;
  const int cc = min(c, ncols - 1);
  const int tok = q0 + cc / H, head = cc % H;
  const int pos = c < ncols ? start_pos + cc / H : -1;     // -1: an idle column; it sees no key and writes nothing
  bf16x8 qv[KS_C + KS_R];
  {
    const bf16* qp = q + (size_t)tok * q_tok + (size_t)head * q_head + kq * 8;
#pragma unroll
    for (int s = 0; s < KS_C + KS_R; ++s) qv[s] = *reinterpret_cast<const bf16x8*>(qp + s * 32);
  }
  bf16x8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;

  float m = -INFINITY;
  f32x4 lsum = {0.f, 0.f, 0.f, 0.f};
  f32x4 o[CT];
#pragma unroll
  for (int t = 0; t < CT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int base = (key_lo / 32 + wave) * 32; base <= key_hi; base += 32 * LM_WAVES) {
    // the two 16-key halves of the block: a half lies in one page (pages hold a multiple of 16 keys)
    size_t row0[2];     // first key's row in the pools (page * page_size + offset); the null page past the context
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kb = base + u * 16;
      const int page = kb <= key_hi ? __builtin_amdgcn_readfirstlane(table[kb / page_size]) : 0;
      row0[u] = (size_t)page * page_size + (kb <= key_hi ? kb % page_size : 0);
    }
    // scores: s[u] holds keys base + u*16 + kq*4 + (0..3) of this lane's column.  All key fragments of the block are
    // asked for before the first product, so that a block costs one trip to memory for its keys, not one per fragment.
    f32x4 s[2];
    {
      bf16x8 kf[2][KS_C + KS_R];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const bf16* kp = c_pages + (row0[u] + col16) * C + kq * 8;
        const bf16* rp = r_pages + (row0[u] + col16) * R + kq * 8;
#pragma unroll
        for (int ks = 0; ks < KS_C; ++ks) kf[u][ks] = *reinterpret_cast<const bf16x8*>(kp + ks * 32);
#pragma unroll
        for (int ks = 0; ks < KS_R; ++ks) kf[u][KS_C + ks] = *reinterpret_cast<const bf16x8*>(rp + ks * 32);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS_C + KS_R; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][ks], qv[ks], acc, 0, 0, 0);
        s[u] = acc;
      }
    }
    // mask, block maximum
    float bm = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = base + u * 16 + kq * 4 + i;
        const bool see = key <= pos && (window <= 0 || key > pos - window);
        const float v = see ? s[u][i] * scale_log2e : -INFINITY;
        s[u][i] = v;
        bm = fmaxf(bm, v);
      }
    bm = fmaxf(bm, __shfl_xor(bm, 16, MS_WAVE));
    bm = fmaxf(bm, __shfl_xor(bm, 32, MS_WAVE));
    const float m_new = fmaxf(m, bm);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m - m_safe);     // m = -inf: 0
    m = m_new;
    bf16x8 p;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) p[u * 4 + i] = (__bf16)__builtin_amdgcn_exp2f(s[u][i] - m_safe);
    if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
      lsum *= corr;
#pragma unroll
      for (int t = 0; t < CT; ++t) o[t] *= corr;
    }
    lsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p, lsum, 0, 0, 0);
    // values: lane holds entry t*16 + col16 of the latent for keys u*16 + kq*4 + (0..3)
    const bool tail = base + 31 > key_hi;
    const bf16* vp0 = ct_pages + (row0[0] / page_size) * (size_t)page_size * C + row0[0] % page_size + kq * 4;
    const bf16* vp1 = ct_pages + (row0[1] / page_size) * (size_t)page_size * C + row0[1] % page_size + kq * 4;
    constexpr int VG = CT < 16 ? CT : 16;      // tiles of 16 entries whose values are asked for together
#pragma unroll
    for (int t0 = 0; t0 < CT; t0 += VG) {
      bf16x4 va[VG], vb[VG];
#pragma unroll
      for (int j = 0; j < VG; ++j) {
        const size_t at = (size_t)((t0 + j) * 16 + col16) * page_size;
        va[j] = *reinterpret_cast<const bf16x4*>(vp0 + at);
        vb[j] = *reinterpret_cast<const bf16x4*>(vp1 + at);
      }
#pragma unroll
      for (int j = 0; j < VG; ++j) {
        bf16x8 vv;
#pragma unroll
        for (int i = 0; i < 4; ++i) { vv[i] = va[j][i]; vv[4 + i] = vb[j][i]; }
        if (tail) {      // what a reused page still holds past the last visible key must not meet the zero weights
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (base + kq * 4 + i > key_hi) vv[i] = (__bf16)0.0f;
            if (base + 16 + kq * 4 + i > key_hi) vv[4 + i] = (__bf16)0.0f;
          }
        }
        o[t0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, p, o[t0 + j], 0, 0, 0);
      }
    }
  }
  float l = lsum[0];      // every row of the product with ones is the column's sum
  // merge the waves' shares (each relative to its own maximum) into wave 0, in wave order
  if (kq == 0) { sm_m[wave][col16] = m; sm_l[wave][col16] = l; }
  __syncthreads();
  {
    float big = sm_m[0][col16];
#pragma unroll
    for (int w = 1; w < LM_WAVES; ++w) big = fmaxf(big, sm_m[w][col16]);
    const float safe = big == -INFINITY ? 0.f : big;
    const float f = __builtin_amdgcn_exp2f(m - safe);      // a wave that saw no key: 0
#pragma unroll
    for (int t = 0; t < CT; ++t) o[t] *= f;
    l = 0.f;
#pragma unroll
    for (int w = 0; w < LM_WAVES; ++w) l += sm_l[w][col16] * __builtin_amdgcn_exp2f(sm_m[w][col16] - safe);
    m = big;
  }
  for (int w = 1; w < LM_WAVES; ++w) {
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < CT; ++t) sm_o[t][lane] = o[t];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < CT; ++t) o[t] += sm_o[t][lane];
    }
    __syncthreads();
  }
  if (wave != 0 || pos < 0) return;
  if (sink) {             // the sink: one more term exp(sink) in the denominator, unscaled, with no value
    const float sk = sink[head] * 1.4426950408889634f;
    const float big = fmaxf(m, sk);
    const float f = __builtin_amdgcn_exp2f(m - big);
    l = l * f + __builtin_amdgcn_exp2f(sk - big);
#pragma unroll
    for (int t = 0; t < CT; ++t) o[t] *= f;
  }
  const float inv = 1.0f / l;
  bf16* op = out + (size_t)tok * out_tok + (size_t)head * out_head + kq * 4;
#pragma unroll
  for (int t = 0; t < CT; ++t) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (__bf16)(o[t][i] * inv);
    *reinterpret_cast<bf16x4*>(op + t * 16) = w;
  }
}

// The shape for long portions: the four waves of a block own four neighbouring tiles (64 columns, whose key ranges
// all but coincide) and read every key block from LDS, where the block's threads have put it together once: the
// keys as rows of C + R entries, the transposed latents as rows of 32 keys, both padded so that the fragments'
// reads spread over the banks.  A key block then comes from the L2 once for 64 columns instead of once for 16.
constexpr int LS_KPAD = 8, LS_VROW = 40;     // entries: a key's row is C + R + 8 long, a latent entry's row 32 + 8

template <int C, int R>
__global__ void __launch_bounds__(LM_WAVES * MS_WAVE)
latent_attention_mfma_shared_kernel(const bf16* __restrict__ q, size_t q_tok, size_t q_head,
                                    const bf16* __restrict__ c_pages, const bf16* __restrict__ r_pages,
                                    const bf16* __restrict__ ct_pages, const int* __restrict__ block_table,
                                    int table_stride, const int* __restrict__ table_rows,
                                    const int* __restrict__ q_start, const int* __restrict__ context_lens,
                                    const float* __restrict__ sink, bf16* __restrict__ out, size_t out_tok,
                                    size_t out_head, int H, int page_size, float scale_log2e, int window) {
  constexpr int KS_C = C / 32, KS_R = R / 32, CT = C / 16, KROW = C + R + LS_KPAD;
  extern __shared__ __align__(16) bf16 ls[];
  bf16* Ks = ls;                       // [32][KROW]
  bf16* Vs = ls + 32 * KROW;           // [C][LS_VROW]
  const int lane = threadIdx.x & (MS_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / MS_WAVE);
  const int col16 = lane & 15, kq = lane >> 4;
  const int r = blockIdx.y;
  const int q0 = q_start[r];
  const int qlen = q_start[r + 1] - q0;
  const int ncols = qlen * H;
  const int b0 = blockIdx.x * 16 * LM_WAVES;        // the block's first column
  if (b0 >= ncols) return;                         // the whole block
  const int start_pos = context_lens[r] - qlen;
  const int* table = block_table + (size_t)(table_rows ? table_rows[r] : r) * table_stride;
  // the block's keys: from the first column's window to the last column's own position
  const int blk_hi = start_pos + (min(ncols, b0 + 16 * LM_WAVES) - 1) / H;
  const int blk_lo = window > 0 ? max(0, start_pos + b0 / H - window + 1) : 0;
  // this wave's tile and this lane's column
  const int c0 = b0 + wave * 16;
  const bool tile = c0 < ncols;
  const int last_col = min(ncols, c0 + 16) - 1;
  const int key_hi = tile ? start_pos + last_col / H : -1;
  const int key_lo = (tile && window > 0) ? max(0, start_pos + c0 / H - window + 1) : 0;
  const int c = c0 + col16;
  const int cc = min(c, ncols - 1);
  const int tok = q0 + cc / H, head = cc % H;
  const int pos = c < ncols ? start_pos + cc / H : -1;
  bf16x8 qv[KS_C + KS_R];
  {
    const bf16* qp = q + (size_t)tok * q_tok + (size_t)head * q_head + kq * 8;
#pragma unroll
    for (int s = 0; s < KS_C + KS_R; ++s) qv[s] = *reinterpret_cast<const bf16x8*>(qp + s * 32);
  }
  bf16x8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;
  float m = -INFINITY;
  f32x4 lsum = {0.f, 0.f, 0.f, 0.f};
  f32x4 o[CT];
#pragma unroll
  for (int t = 0; t < CT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  constexpr int KSEG = (C + R) / 8;     // pieces of 16 bytes in a key's row
  constexpr int THREADS = LM_WAVES * MS_WAVE;
  constexpr int KPT = (32 * KSEG + THREADS - 1) / THREADS, VPT = C * 4 / THREADS;   // pieces a thread carries
  // A key block is asked for one block ahead, into registers, and its page ids one block before that: while a block is
  // multiplied the next one is on its way, and no load waits for a look-up.
  bf16x8 kreg[KPT], vreg[VPT];
  int pages[2];
  auto lookup = [&](int base) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kb = base + u * 16;
      pages[u] = kb <= blk_hi ? __builtin_amdgcn_readfirstlane(table[kb / page_size]) : 0;
    }
  };
  auto issue = [&](int base) __attribute__((always_inline)) {
    size_t row0[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) row0[u] = (size_t)pages[u] * page_size + (base + u * 16 <= blk_hi ? (base + u * 16) % page_size : 0);
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
      const int seg = threadIdx.x + j * THREADS;
      if (seg < 32 * KSEG) {
        const int key = seg / KSEG, piece = seg - key * KSEG;
        const size_t row = row0[key >> 4] + (key & 15);
        const bf16* src = piece < C / 8 ? c_pages + row * C + piece * 8 : r_pages + row * R + (piece - C / 8) * 8;
        kreg[j] = *reinterpret_cast<const bf16x8*>(src);
      }
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int seg = threadIdx.x + j * THREADS;
      const int u = seg / (C * 2), rem = seg - u * (C * 2), dim = rem >> 1, piece = rem & 1;
      const bf16* src = ct_pages + (row0[u] / page_size) * (size_t)page_size * C + (size_t)dim * page_size +
                        row0[u] % page_size + piece * 8;
      vreg[j] = *reinterpret_cast<const bf16x8*>(src);
    }
  };
  auto commit = [&](int base) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
      const int seg = threadIdx.x + j * THREADS;
      if (seg < 32 * KSEG) {
        const int key = seg / KSEG, piece = seg - key * KSEG;
        *reinterpret_cast<bf16x8*>(Ks + key * KROW + piece * 8) = kreg[j];
      }
    }
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int seg = threadIdx.x + j * THREADS;
      const int u = seg / (C * 2), rem = seg - u * (C * 2), dim = rem >> 1, piece = rem & 1;
      bf16x8 v = vreg[j];
      // what a reused page still holds past the block's last key must not meet the zero weights
      const int k0 = base + u * 16 + piece * 8;
      if (k0 + 7 > blk_hi) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (k0 + i > blk_hi) v[i] = (__bf16)0.0f;
      }
      *reinterpret_cast<bf16x8*>(Vs + dim * LS_VROW + u * 16 + piece * 8) = v;
    }
  };
  constexpr bool AHEAD = C <= 256;      // at 512 the accumulators and the query leave no registers to carry a block
  const int first = (blk_lo / 32) * 32;
  lookup(first);
  if (AHEAD) {
    issue(first);
    if (first + 32 <= blk_hi) lookup(first + 32);
  }
  for (int base = first; base <= blk_hi; base += 32) {
    __syncthreads();     // everyone is done with the block before
    if (AHEAD) {
      commit(base);
    } else {
      // four pieces in flight at a time, straight into LDS
      size_t row0[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) row0[u] = (size_t)pages[u] * page_size + (base + u * 16 <= blk_hi ? (base + u * 16) % page_size : 0);
      if (base + 32 <= blk_hi) lookup(base + 32);     // the next block's page ids travel with this block's keys
      constexpr int G = 4;
#pragma unroll
      for (int j0 = 0; j0 < KPT; j0 += G) {
        bf16x8 t[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int seg = threadIdx.x + (j0 + g) * THREADS;
          if (j0 + g < KPT && seg < 32 * KSEG) {
            const int key = seg / KSEG, piece = seg - key * KSEG;
            const size_t row = row0[key >> 4] + (key & 15);
            t[g] = *reinterpret_cast<const bf16x8*>(piece < C / 8 ? c_pages + row * C + piece * 8
                                                                  : r_pages + row * R + (piece - C / 8) * 8);
          }
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int seg = threadIdx.x + (j0 + g) * THREADS;
          if (j0 + g < KPT && seg < 32 * KSEG) {
            const int key = seg / KSEG, piece = seg - key * KSEG;
            *reinterpret_cast<bf16x8*>(Ks + key * KROW + piece * 8) = t[g];
          }
        }
      }
#pragma unroll
      for (int j0 = 0; j0 < VPT; j0 += G) {
        bf16x8 t[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          if (j0 + g < VPT) {
            const int seg = threadIdx.x + (j0 + g) * THREADS;
            const int u = seg / (C * 2), rem = seg - u * (C * 2), dim = rem >> 1, piece = rem & 1;
            t[g] = *reinterpret_cast<const bf16x8*>(ct_pages + (row0[u] / page_size) * (size_t)page_size * C +
                                                    (size_t)dim * page_size + row0[u] % page_size + piece * 8);
          }
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          if (j0 + g < VPT) {
            const int seg = threadIdx.x + (j0 + g) * THREADS;
            const int u = seg / (C * 2), rem = seg - u * (C * 2), dim = rem >> 1, piece = rem & 1;
            bf16x8 v = t[g];
            const int k0 = base + u * 16 + piece * 8;
            if (k0 + 7 > blk_hi) {
#pragma unroll
              for (int i = 0; i < 8; ++i)
                if (k0 + i > blk_hi) v[i] = (__bf16)0.0f;
            }
            *reinterpret_cast<bf16x8*>(Vs + dim * LS_VROW + u * 16 + piece * 8) = v;
          }
        }
      }
    }
    __syncthreads();
    if (AHEAD && base + 32 <= blk_hi) {
      issue(base + 32);
      if (base + 64 <= blk_hi) lookup(base + 64);
    }
    if (!tile || base > key_hi || base + 31 < key_lo) continue;     // none of this block's keys is the tile's
    f32x4 s[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const bf16* kp = Ks + (u * 16 + col16) * KROW + kq * 8;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS_C + KS_R; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(kp + ks * 32), qv[ks], acc, 0, 0, 0);
      s[u] = acc;
    }
    float bm = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = base + u * 16 + kq * 4 + i;
        const bool see = key <= pos && (window <= 0 || key > pos - window);
        const float v = see ? s[u][i] * scale_log2e : -INFINITY;
        s[u][i] = v;
        bm = fmaxf(bm, v);
      }
    bm = fmaxf(bm, __shfl_xor(bm, 16, MS_WAVE));
    bm = fmaxf(bm, __shfl_xor(bm, 32, MS_WAVE));
    const float m_new = fmaxf(m, bm);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m - m_safe);
    m = m_new;
    bf16x8 p;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) p[u * 4 + i] = (__bf16)__builtin_amdgcn_exp2f(s[u][i] - m_safe);
    if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
      lsum *= corr;
#pragma unroll
      for (int t = 0; t < CT; ++t) o[t] *= corr;
    }
    lsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p, lsum, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < CT; ++t) {
      const bf16* vp = Vs + (t * 16 + col16) * LS_VROW + kq * 4;
      const bf16x4 a = *reinterpret_cast<const bf16x4*>(vp);
      const bf16x4 b = *reinterpret_cast<const bf16x4*>(vp + 16);
      bf16x8 vv;
#pragma unroll
      for (int i = 0; i < 4; ++i) { vv[i] = a[i]; vv[4 + i] = b[i]; }
      o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, p, o[t], 0, 0, 0);
    }
  }
  if (pos < 0) return;
  float l = lsum[0];
  if (sink) {
    const float sk = sink[head] * 1.4426950408889634f;
    const float big = fmaxf(m, sk);
    const float f = __builtin_amdgcn_exp2f(m - big);
    l = l * f + __builtin_amdgcn_exp2f(sk - big);
#pragma unroll
    for (int t = 0; t < CT; ++t) o[t] *= f;
  }
  const float inv = 1.0f / l;
  bf16* op = out + (size_t)tok * out_tok + (size_t)head * out_head + kq * 4;
#pragma unroll
  for (int t = 0; t < CT; ++t) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (__bf16)(o[t][i] * inv);
    *reinterpret_cast<bf16x4*>(op + t * 16) = w;
  }
}

}  // namespace

extern "C" int ms_latent_attention_mfma_supported(int C, int R, int page_size) {
  return (C == 128 || C == 256 || C == 512) && (R == 32 || R == 64) && page_size > 0 && page_size % 16 == 0;
}

// q [n, heads, C + R] (strides in elements, 16-byte aligned rows), c_pages [P, 1, page, C], r_pages [P, 1, page, R],
// ct_pages [P, 1, C, page] (the latents once more, transposed), out [n, heads, C].  Request r owns tokens
// q_start[r]..q_start[r+1]-1 and holds context_lens[r] keys once this step's are stored; max_q_len bounds its tokens.
extern "C" int ms_latent_attention_mfma(const void* q, long long q_tok, long long q_head, const void* c_pages,
                                        const void* r_pages, const void* ct_pages, const int* block_table,
                                        int table_stride, const int* table_rows, const int* q_start,
                                        const int* context_lens, const float* sink, void* out, long long out_tok,
                                        long long out_head, int n_requests, int max_q_len, int heads, int C, int R,
                                        int page_size, long long num_pages, float scale, int window,
                                        hipStream_t stream) {
  if (n_requests <= 0 || max_q_len <= 0) return MS_OK;
  if (heads <= 0 || table_stride <= 0) return MS_BAD_ARG;
  if (!ms_latent_attention_mfma_supported(C, R, page_size)) return MS_UNSUPPORTED;
  if (q_tok % 8 || q_head % 8 || out_tok % 4 || out_head % 4) return MS_UNSUPPORTED;
  if (num_pages * page_size >= (1ll << 31) || n_requests > 65535) return MS_UNSUPPORTED;
  const long long tiles = ((long long)max_q_len * heads + 15) / 16;
  const float sl = scale * 1.4426950408889634f;
  // long portions: four neighbouring tiles a block over key blocks staged in LDS (more than the 64 KB a launch may
  // ask for without more ado, so the kernel's limit is raised once); else a tile's keys over the four waves
  const size_t shared_lds = ((size_t)32 * (C + R + LS_KPAD) + (size_t)C * LS_VROW) * sizeof(bf16);
  const bool shared = tiles >= 8;
  dim3 grid((unsigned)(shared ? (tiles + LM_WAVES - 1) / LM_WAVES : tiles), n_requests), block(LM_WAVES * MS_WAVE);
#define ARGS                                                                                                            \
      (const bf16*)q, (size_t)q_tok, (size_t)q_head, (const bf16*)c_pages, (const bf16*)r_pages, (const bf16*)ct_pages, \
      block_table, table_stride, table_rows, q_start, context_lens, sink, (bf16*)out, (size_t)out_tok,                  \
      (size_t)out_head, heads, page_size, sl, window
#define LAUNCH(CC, RR)                                                                                                  \
  do {                                                                                                                  \
    if (shared) {                                                                                                       \
      static bool raised = false;                                                                                       \
      if (!raised) {                                                                                                    \
        if (hipFuncSetAttribute((const void*)latent_attention_mfma_shared_kernel<CC, RR>,                               \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shared_lds) != hipSuccess)             \
          return MS_LAUNCH_FAILED;                                                                                      \
        raised = true;                                                                                                  \
      }                                                                                                                 \
      latent_attention_mfma_shared_kernel<CC, RR><<<grid, block, shared_lds, stream>>>(ARGS);                           \
    } else {                                                                                                            \
      latent_attention_mfma_kernel<CC, RR><<<grid, block, 0, stream>>>(ARGS);                                           \
    }                                                                                                                   \
  } while (0)
  if (C == 128 && R == 32) LAUNCH(128, 32);
  else if (C == 128 && R == 64) LAUNCH(128, 64);
  else if (C == 256 && R == 32) LAUNCH(256, 32);
  else if (C == 256 && R == 64) LAUNCH(256, 64);
  else if (C == 512 && R == 32) LAUNCH(512, 32);
  else LAUNCH(512, 64);
#undef LAUNCH
#undef ARGS
  return ms_launch_status();
}
