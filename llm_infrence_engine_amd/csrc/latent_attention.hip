// Attention through a low-rank latent.  A token's cache entry is its normalised latent c [C] and one rotated
// key part kr [R] shared by all heads; keys and values of the heads are linear maps of c, so a head's score
// against key j is (W_uk^T q_flat) . c_j + q_rot . kr_j and its output W_uv (sum_j p_j c_j): the maps move to the
// query and to the output and the attention itself runs over the cached latents alone, as one key/value "head"
// that every query head reads.
//   ms_head_matmul      out[n, h, :] = in[n, h, :] @ M[h]  (the two per-head maps), optionally gated
//   ms_rotary_pairs     rotation of neighbouring pairs (2i, 2i+1) by position * inv_freq[i], copying the rest
//   ms_latent_kv_store  RMS norm of the latent, rotation of the shared key part, both into their pages
//   ms_latent_attention sliding-window softmax attention over the pages with a per-head sink in the denominator
// Scores, softmax, norms and angles are float in every mode.
#include "common.h"
#include "api.h"

namespace {

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ------------------------------------------------------------------------------------------------
// out[n, h, j] = sum_i in[n, h, i] * M[h, i, j] (* sigmoid(gate[n, h, j])).  A block owns TM tokens of one head and 64
// consecutive j; its four waves each take a quarter of the i (rows of M, read coalesced, eight in flight) and their
// sums are added through LDS in wave order: the shape for few tokens (a decode step), where blocks are few and a
// thread's walk over all the i would be the longest chain of the step.
constexpr int HM_WAVES = 4;

template <typename T, typename TO, int TM>
__global__ void __launch_bounds__(HM_WAVES * MS_WAVE)
head_matmul_kernel(const T* __restrict__ in, size_t in_tok, size_t in_head, const T* __restrict__ M,
                   TO* __restrict__ out, size_t out_tok, size_t out_head, const T* __restrict__ gate,
                   size_t gate_tok, int N, int I, int J) {
  extern __shared__ __align__(16) float xs[];   // [I][TM], then [HM_WAVES - 1][TM][64] for the waves' sums
  float* part = xs + (size_t)I * TM;
  const int h = blockIdx.y, n0 = blockIdx.x * TM;
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const int j = blockIdx.z * MS_WAVE + lane;
  for (int e = threadIdx.x; e < I * TM; e += blockDim.x) {
    const int t = e / I, i = e - t * I;
    xs[i * TM + t] = n0 + t < N ? to_float(in[(size_t)(n0 + t) * in_tok + (size_t)h * in_head + i]) : 0.f;
  }
  __syncthreads();
  float acc[TM];
#pragma unroll
  for (int t = 0; t < TM; ++t) acc[t] = 0.f;
  const int per = (I + HM_WAVES - 1) / HM_WAVES;
  const int i0 = wave * per, i1 = min(I, i0 + per);
  if (j < J) {
    const T* Mh = M + (size_t)h * I * J + j;
#pragma unroll 32
    for (int i = i0; i < i1; ++i) {   // thirty-two rows of M in flight: with few blocks a wave's trips to memory are the time
      const float m = to_float(Mh[(size_t)i * J]);
#pragma unroll
      for (int t = 0; t < TM; t += 4) {
        const float4 a = *reinterpret_cast<const float4*>(xs + i * TM + t);
        acc[t] = fmaf(a.x, m, acc[t]); acc[t + 1] = fmaf(a.y, m, acc[t + 1]);
        acc[t + 2] = fmaf(a.z, m, acc[t + 2]); acc[t + 3] = fmaf(a.w, m, acc[t + 3]);
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < TM; ++t) part[((wave - 1) * TM + t) * MS_WAVE + lane] = acc[t];
  }
  __syncthreads();
  if (wave > 0 || j >= J) return;
#pragma unroll
  for (int t = 0; t < TM; ++t) {
    if (n0 + t >= N) break;
    float y = acc[t];
    for (int w = 0; w < HM_WAVES - 1; ++w) y += part[(w * TM + t) * MS_WAVE + lane];
    if (gate) y *= sigmoid_f(to_float(gate[(size_t)(n0 + t) * gate_tok + (size_t)h * J + j]));
    out[(size_t)(n0 + t) * out_tok + (size_t)h * out_head + j] = from_float<TO>(y);
  }
}

// The same product for many tokens: a block owns 8 tokens of one head and up to 256 consecutive j, a thread all the i
// of its j; the blocks are many, and each reads its tokens once.
constexpr int HM_TOKENS = 8;

template <typename T, typename TO>
__global__ void head_matmul_wide_kernel(const T* __restrict__ in, size_t in_tok, size_t in_head, const T* __restrict__ M,
                                        TO* __restrict__ out, size_t out_tok, size_t out_head, const T* __restrict__ gate,
                                        size_t gate_tok, int N, int I, int J) {
  extern __shared__ __align__(16) float xs[];   // [I][HM_TOKENS]
  const int h = blockIdx.y, n0 = blockIdx.x * HM_TOKENS;
  const int j = blockIdx.z * blockDim.x + threadIdx.x;
  for (int e = threadIdx.x; e < I * HM_TOKENS; e += blockDim.x) {
    const int t = e / I, i = e - t * I;
    xs[i * HM_TOKENS + t] = n0 + t < N ? to_float(in[(size_t)(n0 + t) * in_tok + (size_t)h * in_head + i]) : 0.f;
  }
  __syncthreads();
  if (j >= J) return;
  float acc[HM_TOKENS];
#pragma unroll
  for (int t = 0; t < HM_TOKENS; ++t) acc[t] = 0.f;
  const T* Mh = M + (size_t)h * I * J + j;
#pragma unroll 8
  for (int i = 0; i < I; ++i) {   // eight rows of M in flight: the loop waits for memory, not for arithmetic
    const float m = to_float(Mh[(size_t)i * J]);
    const float4 a = *reinterpret_cast<const float4*>(xs + i * HM_TOKENS);
    const float4 b = *reinterpret_cast<const float4*>(xs + i * HM_TOKENS + 4);
    acc[0] = fmaf(a.x, m, acc[0]); acc[1] = fmaf(a.y, m, acc[1]); acc[2] = fmaf(a.z, m, acc[2]); acc[3] = fmaf(a.w, m, acc[3]);
    acc[4] = fmaf(b.x, m, acc[4]); acc[5] = fmaf(b.y, m, acc[5]); acc[6] = fmaf(b.z, m, acc[6]); acc[7] = fmaf(b.w, m, acc[7]);
  }
#pragma unroll
  for (int t = 0; t < HM_TOKENS; ++t) {
    if (n0 + t >= N) break;
    float y = acc[t];
    if (gate) y *= sigmoid_f(to_float(gate[(size_t)(n0 + t) * gate_tok + (size_t)h * J + j]));
    out[(size_t)(n0 + t) * out_tok + (size_t)h * out_head + j] = from_float<TO>(y);
  }
}

// ------------------------------------------------------------------------------------------------
// dst[n, h, 0:width] = src[n, h, 0:width] with the first `dims` entries turned pair by pair:
// (u, v) = entries (2i, 2i+1) -> (u cos a - v sin a, v cos a + u sin a), a = float(position) * inv_freq[i].
template <typename T>
__global__ void rotary_pairs_kernel(const T* __restrict__ src, size_t src_tok, size_t src_head, T* __restrict__ dst,
                                    size_t dst_tok, size_t dst_head, const int* __restrict__ positions,
                                    const float* __restrict__ inv_freq, int heads, int width, int dims) {
  const int n = blockIdx.x;
  const float pos = (float)positions[n];
  const int half = width / 2 + (width & 1);   // pairs, and a last single entry if the width is odd
  for (int e = threadIdx.x; e < heads * half; e += blockDim.x) {
    const int h = e / half, i = e - h * half;
    const T* s = src + (size_t)n * src_tok + (size_t)h * src_head;
    T* d = dst + (size_t)n * dst_tok + (size_t)h * dst_head;
    if (2 * i + 1 >= width) { d[2 * i] = s[2 * i]; continue; }
    const float u = to_float(s[2 * i]), v = to_float(s[2 * i + 1]);
    if (2 * i + 1 < dims) {
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      d[2 * i] = from_float<T>(u * cs - v * sn);
      d[2 * i + 1] = from_float<T>(v * cs + u * sn);
    } else {
      d[2 * i] = s[2 * i];
      d[2 * i + 1] = s[2 * i + 1];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// out[n, :] = in[n, :] / sqrt(mean(in[n, :]^2) + eps) * w: the norm of an activation (not of the residual stream).
template <typename T>
__global__ void rms_norm_rows_kernel(const T* __restrict__ in, size_t in_stride, const float* __restrict__ w,
                                     T* __restrict__ out, size_t out_stride, int C, float eps) {
  __shared__ float red[16];
  const T* x = in + (size_t)blockIdx.x * in_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += blockDim.x) { const float v = to_float(x[i]); ss = fmaf(v, v, ss); }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)C + eps);
  T* o = out + (size_t)blockIdx.x * out_stride;
  for (int i = threadIdx.x; i < C; i += blockDim.x) o[i] = from_float<T>(to_float(x[i]) * inv * w[i]);
}

// ------------------------------------------------------------------------------------------------
// kv [N, C + R]: c = rms_norm(kv[:, :C]) * w -> latent pages at the token's slot; kv[:, C:] rotated -> key-part pages.
// Pages are [page][slot][entry] with one head.
template <typename T>
__global__ void latent_kv_store_kernel(const T* __restrict__ kv, size_t kv_stride, const float* __restrict__ w, float eps,
                                       const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                       const int* __restrict__ slots, T* __restrict__ c_pages, T* __restrict__ r_pages,
                                       T* __restrict__ ct_pages, int page_size, int C, int R, int dims) {
  __shared__ float red[16];
  const int n = blockIdx.x;
  const int slot = slots[n];
  if (slot < 0) return;        // uniform for the block: a token that stores nothing
  const T* x = kv + (size_t)n * kv_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < C; i += blockDim.x) { const float v = to_float(x[i]); ss = fmaf(v, v, ss); }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)C + eps);
  T* cp = c_pages + (size_t)slot * C;
  // ct_pages (may be null): the same latents once more as [page][entry][slot], for kernels that read them as a
  // matrix operand with the keys along a row
  T* tp = ct_pages ? ct_pages + (size_t)(slot / page_size) * page_size * C + slot % page_size : nullptr;
  for (int i = threadIdx.x; i < C; i += blockDim.x) {
    const T v = from_float<T>(to_float(x[i]) * inv * w[i]);
    cp[i] = v;
    if (tp) tp[(size_t)i * page_size] = v;
  }
  const float pos = (float)positions[n];
  T* rp = r_pages + (size_t)slot * R;
  const T* xr = x + C;
  for (int i = threadIdx.x; i < (R + 1) / 2; i += blockDim.x) {
    if (2 * i + 1 >= R) { rp[2 * i] = xr[2 * i]; continue; }
    const float u = to_float(xr[2 * i]), v = to_float(xr[2 * i + 1]);
    if (2 * i + 1 < dims) {
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      rp[2 * i] = from_float<T>(u * cs - v * sn);
      rp[2 * i + 1] = from_float<T>(v * cs + u * sn);
    } else {
      rp[2 * i] = xr[2 * i];
      rp[2 * i + 1] = xr[2 * i + 1];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// One wave per (token, head): q [C + R] (the mapped flat part, then the rotated part), keys [c_j ; kr_j] read in
// place through the request's block table, values c_j.  The sink is where the running maximum and sum start:
// m = sink, l = 1, nothing accumulated; it is not scaled and has no value.
constexpr int LA_WAVES = 4;
constexpr int LA_MAX_C = 1024;

template <typename T>
__global__ void __launch_bounds__(LA_WAVES * MS_WAVE)
latent_attention_kernel(const T* __restrict__ q, size_t q_tok, size_t q_head, const T* __restrict__ c_pages,
                        const T* __restrict__ r_pages, const int* __restrict__ block_table, int table_stride,
                        const int* __restrict__ table_rows, const int* __restrict__ n_live_tokens,
                        const int* __restrict__ token_req, const int* __restrict__ positions,
                        const float* __restrict__ sink, T* __restrict__ out, size_t out_tok, size_t out_head,
                        int n_tokens, int H, int C, int R, int page_size, float scale, int window) {
  extern __shared__ __align__(16) float qs_all[];   // [LA_WAVES][C + R]
  const int lane = threadIdx.x & (MS_WAVE - 1), wave = threadIdx.x / MS_WAVE;
  const long long item = (long long)blockIdx.x * LA_WAVES + wave;
  if (item >= (long long)n_tokens * H) return;   // whole wave leaves; no block-wide barrier below
  const int n = (int)(item / H), h = (int)(item - (long long)n * H);
  if (n_live_tokens && n >= *n_live_tokens) return;
  const int pos = positions[n];
  const int req = token_req[n];
  const int* table = block_table + (size_t)(table_rows ? table_rows[req] : req) * table_stride;
  float* qs = qs_all + (size_t)wave * (C + R);
  const T* qp = q + (size_t)n * q_tok + (size_t)h * q_head;
  for (int i = lane; i < C + R; i += MS_WAVE) qs[i] = to_float(qp[i]) * scale;
  __builtin_amdgcn_wave_barrier();

  int start = 0;
  if (window > 0 && pos - window + 1 > 0) start = pos - window + 1;
  float m = sink ? sink[h] : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[LA_MAX_C / MS_WAVE];
#pragma unroll
  for (int c = 0; c < LA_MAX_C / MS_WAVE; ++c) acc[c] = 0.f;

  for (int base = start; base <= pos; base += MS_WAVE) {
    const int j = base + lane;
    const bool valid = j <= pos;
    int row = 0;
    float s = -INFINITY;
    if (valid) {
      row = table[j / page_size] * page_size + (j % page_size);
      const T* cp = c_pages + (size_t)row * C;
      const T* rp = r_pages + (size_t)row * R;
      float dot = 0.f;
      for (int i = 0; i < C; ++i) dot = fmaf(qs[i], to_float(cp[i]), dot);
      for (int i = 0; i < R; ++i) dot = fmaf(qs[C + i], to_float(rp[i]), dot);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);   // 0 while m is still -inf and m_new finite
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < LA_MAX_C / MS_WAVE; ++c) acc[c] *= corr;
    const int count = min(MS_WAVE, pos - base + 1);
    for (int jj = 0; jj < count; ++jj) {
      const float pj = __shfl(p, jj, MS_WAVE);
      const int vrow = __shfl(row, jj, MS_WAVE);
      const T* vp = c_pages + (size_t)vrow * C;
#pragma unroll
      for (int c = 0; c < LA_MAX_C / MS_WAVE; ++c) {
        const int i = lane + c * MS_WAVE;
        if (i < C) acc[c] = fmaf(pj, to_float(vp[i]), acc[c]);
      }
    }
  }
  T* op = out + (size_t)n * out_tok + (size_t)h * out_head;
  const float inv = 1.0f / l;
#pragma unroll
  for (int c = 0; c < LA_MAX_C / MS_WAVE; ++c) {
    const int i = lane + c * MS_WAVE;
    if (i < C) op[i] = from_float<T>(acc[c] * inv);
  }
}

}  // namespace

extern "C" int ms_head_matmul(const void* in, long long in_tok, long long in_head, const void* M, void* out,
                              long long out_tok, long long out_head, const void* gate, long long gate_tok, int n_tokens,
                              int heads, int I, int J, int dtype, int out_dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (heads <= 0 || I <= 0 || J <= 0) return MS_BAD_ARG;
  // float: always the one order of summation, whatever the step holds
  if (n_tokens > 64 || dtype == MS_F32) {
    const size_t lds = (size_t)I * HM_TOKENS * sizeof(float);
    if (lds > 65536 || heads > 65535) return MS_UNSUPPORTED;
    const int threads = J >= 256 ? 256 : ((J + MS_WAVE - 1) / MS_WAVE) * MS_WAVE;
    dim3 grid((n_tokens + HM_TOKENS - 1) / HM_TOKENS, heads, (J + threads - 1) / threads), block(threads);
#define LAUNCH(T, TO) head_matmul_wide_kernel<T, TO><<<grid, block, lds, stream>>>((const T*)in, (size_t)in_tok, (size_t)in_head, (const T*)M, (TO*)out, (size_t)out_tok, (size_t)out_head, (const T*)gate, (size_t)gate_tok, n_tokens, I, J)
    if (dtype == MS_F32 && out_dtype == MS_F32) LAUNCH(float, float);
    else if (dtype == MS_BF16 && out_dtype == MS_BF16) LAUNCH(bf16, bf16);
    else if (dtype == MS_BF16 && out_dtype == MS_F32) LAUNCH(bf16, float);
    else return MS_BAD_ARG;
#undef LAUNCH
    return ms_launch_status();
  }
  constexpr int tm = 8;
  const size_t lds = ((size_t)I * tm + (size_t)(HM_WAVES - 1) * tm * MS_WAVE) * sizeof(float);
  if (lds > 65536 || heads > 65535 || (J + MS_WAVE - 1) / MS_WAVE > 65535) return MS_UNSUPPORTED;
  dim3 grid((n_tokens + tm - 1) / tm, heads, (J + MS_WAVE - 1) / MS_WAVE), block(HM_WAVES * MS_WAVE);
#define LAUNCH(T, TO) head_matmul_kernel<T, TO, 8><<<grid, block, lds, stream>>>((const T*)in, (size_t)in_tok, (size_t)in_head, (const T*)M, (TO*)out, (size_t)out_tok, (size_t)out_head, (const T*)gate, (size_t)gate_tok, n_tokens, I, J)
  if (dtype == MS_F32 && out_dtype == MS_F32) LAUNCH(float, float);
  else if (dtype == MS_BF16 && out_dtype == MS_BF16) LAUNCH(bf16, bf16);
  else if (dtype == MS_BF16 && out_dtype == MS_F32) LAUNCH(bf16, float);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

extern "C" int ms_rms_norm_rows(const void* in, long long in_stride, const float* weight, void* out, long long out_stride,
                                int n_rows, int width, float eps, int dtype, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (width <= 0) return MS_BAD_ARG;
  dim3 grid(n_rows), block(width >= 512 ? 256 : 128);
  if (dtype == MS_F32)
    rms_norm_rows_kernel<float><<<grid, block, 0, stream>>>((const float*)in, (size_t)in_stride, weight, (float*)out,
                                                            (size_t)out_stride, width, eps);
  else if (dtype == MS_BF16)
    rms_norm_rows_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)in, (size_t)in_stride, weight, (bf16*)out,
                                                           (size_t)out_stride, width, eps);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_rotary_pairs(const void* src, long long src_tok, long long src_head, void* dst, long long dst_tok,
                               long long dst_head, const int* positions, const float* inv_freq, int n_tokens, int heads,
                               int width, int dims, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (heads <= 0 || width <= 0 || dims < 0 || dims > width || dims % 2) return MS_BAD_ARG;
  dim3 grid(n_tokens), block(256);
  if (dtype == MS_F32)
    rotary_pairs_kernel<float><<<grid, block, 0, stream>>>((const float*)src, (size_t)src_tok, (size_t)src_head, (float*)dst,
                                                           (size_t)dst_tok, (size_t)dst_head, positions, inv_freq, heads, width, dims);
  else if (dtype == MS_BF16)
    rotary_pairs_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)src, (size_t)src_tok, (size_t)src_head, (bf16*)dst,
                                                          (size_t)dst_tok, (size_t)dst_head, positions, inv_freq, heads, width, dims);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_latent_kv_store(const void* kv, long long kv_stride, const float* norm_w, float eps, const int* positions,
                                  const float* inv_freq, const int* slots, void* c_pages, void* r_pages, void* ct_pages,
                                  int page_size, int n_tokens, int C, int R, int dims, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (C <= 0 || R <= 0 || dims < 0 || dims > R || dims % 2 || page_size <= 0) return MS_BAD_ARG;
  dim3 grid(n_tokens), block(C >= 512 ? 256 : 128);
  if (dtype == MS_F32)
    latent_kv_store_kernel<float><<<grid, block, 0, stream>>>((const float*)kv, (size_t)kv_stride, norm_w, eps, positions, inv_freq,
                                                              slots, (float*)c_pages, (float*)r_pages, (float*)ct_pages, page_size, C, R, dims);
  else if (dtype == MS_BF16)
    latent_kv_store_kernel<bf16><<<grid, block, 0, stream>>>((const bf16*)kv, (size_t)kv_stride, norm_w, eps, positions, inv_freq,
                                                             slots, (bf16*)c_pages, (bf16*)r_pages, (bf16*)ct_pages, page_size, C, R, dims);
  else return MS_BAD_ARG;
  return ms_launch_status();
}

extern "C" int ms_latent_attention(const void* q, long long q_tok, long long q_head, const void* c_pages, const void* r_pages,
                                   const int* block_table, int table_stride, const int* table_rows,
                                   const int* n_live_tokens, const int* token_req, const int* positions, const float* sink,
                                   void* out, long long out_tok, long long out_head, int n_tokens, int heads, int C, int R,
                                   int page_size, long long num_pages, float scale, int window, int dtype,
                                   hipStream_t stream) {
  if (n_tokens <= 0) return MS_OK;
  if (heads <= 0 || C <= 0 || R < 0 || page_size <= 0 || table_stride <= 0) return MS_BAD_ARG;
  if (C > LA_MAX_C) return MS_UNSUPPORTED;
  if (num_pages * page_size >= (1ll << 31)) return MS_UNSUPPORTED;   // row index is an int
  const size_t lds = (size_t)LA_WAVES * (C + R) * sizeof(float);
  if (lds > 65536) return MS_UNSUPPORTED;
  const long long items = (long long)n_tokens * heads;
  dim3 grid((unsigned)((items + LA_WAVES - 1) / LA_WAVES)), block(LA_WAVES * MS_WAVE);
#define LAUNCH(T) latent_attention_kernel<T><<<grid, block, lds, stream>>>((const T*)q, (size_t)q_tok, (size_t)q_head, (const T*)c_pages, (const T*)r_pages, block_table, table_stride, table_rows, n_live_tokens, token_req, positions, sink, (T*)out, (size_t)out_tok, (size_t)out_head, n_tokens, heads, C, R, page_size, scale, window)
  if (dtype == MS_F32) LAUNCH(float);
  else if (dtype == MS_BF16) LAUNCH(bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}
