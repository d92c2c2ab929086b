// The selective scan of a state-space mixer.  Per request, channel c and state index n, token by token:
//   dt_c = softplus(dt_in_c + dt_bias_c)
//   S[c, n] <- exp(dt_c * A[c, n]) * S[c, n] + dt_c * x_c * B_n
//   y_c = sum_n S[c, n] * C_n + D_c * x_c;      out_c = y_c * silu(z_c)
// S float [slots, channels, states] is carried from step to step in the request's slot.  A row of S (one channel) is
// held in the registers of LPC neighbouring lanes, SPT states each, for the whole portion.  Tokens are staged a chunk
// at a time: all threads of the block work out the chunk's step sizes (bias, softplus) and convert its x, z, B and C
// into LDS (asked for a chunk ahead), then every thread walks the chunk's tokens in order.  Step sizes, exponentials and the state are float.
// A step is a ragged batch: request r owns the tokens q_start[r] .. q_start[r+1]-1 and the slot state_slots[r];
// requests without tokens are left alone.
#include "common.h"
#include "api.h"

namespace {

constexpr int SCAN_THREADS = 256;
constexpr int SCAN_CHUNK = 16;

__device__ __forceinline__ float scan_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <int CTRL> __device__ __forceinline__ float scan_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// sum over aligned groups of LPC neighbouring lanes, every lane getting the sum
template <int LPC> __device__ __forceinline__ float scan_group_sum(float v) {
  if (LPC >= 2) v += scan_dpp<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  if (LPC >= 4) v += scan_dpp<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  if (LPC >= 8) v += scan_dpp<0x141>(v);    // row_half_mirror
  if (LPC >= 16) v += scan_dpp<0x140>(v);   // row_mirror
  return v;
}

template <typename T, int SPT, int LPC>
__global__ void __launch_bounds__(SCAN_THREADS)
selective_scan_kernel(const T* __restrict__ x, size_t x_stride, const float* __restrict__ dt_in,
                      const float* __restrict__ dt_bias, const float* __restrict__ A, const T* __restrict__ B,
                      const T* __restrict__ C, size_t bc_stride, const float* __restrict__ Dskip,
                      const T* __restrict__ z, size_t z_stride, float* __restrict__ state,
                      const int* __restrict__ q_start, const int* __restrict__ state_slots, T* __restrict__ out,
                      size_t out_stride, int channels, int states) {
  constexpr int CPB = SCAN_THREADS / LPC;    // channels of a block
  constexpr int NP = SPT * LPC;              // padded number of states
  __shared__ float s_dt[SCAN_CHUNK][CPB], s_x[SCAN_CHUNK][CPB], s_z[SCAN_CHUNK][CPB];
  __shared__ float s_b[SCAN_CHUNK][NP], s_c[SCAN_CHUNK][NP];
  const int r = blockIdx.y;
  const int s0 = q_start[r], L = q_start[r + 1] - s0;
  if (L <= 0) return;
  const int tid = threadIdx.x;
  const int part = tid % LPC, ch_local = tid / LPC;
  const int c0 = blockIdx.x * CPB, ch = c0 + ch_local;
  const bool live = ch < channels;
  float* Sg = state + ((size_t)state_slots[r] * channels + (live ? ch : 0)) * states;
  float S[SPT], a[SPT];
#pragma unroll
  for (int i = 0; i < SPT; ++i) {
    const int n = part * SPT + i;
    const bool in = live && n < states;
    S[i] = in ? Sg[n] : 0.f;
    a[i] = in ? A[(size_t)ch * states + n] * 1.4426950408889634f : 0.f;   // exp(dt a) = 2^(dt a log2 e)
  }
  const float dskip = live ? Dskip[ch] : 0.f;
  // Staging.  A thread asks for its share of the next chunk (raw values, into registers) before it walks the current
  // one, so that a chunk's trip to memory is over by the time the chunk before has been walked.
  constexpr int EPT = (SCAN_CHUNK * CPB + SCAN_THREADS - 1) / SCAN_THREADS;   // (token, channel) pairs a thread stages
  constexpr int BPT = (SCAN_CHUNK * NP + SCAN_THREADS - 1) / SCAN_THREADS;    // (token, state) pairs
  float dt_r[EPT];
  T x_r[EPT], z_r[EPT], b_r[BPT], c_r[BPT];
  auto ask = [&](int t0) __attribute__((always_inline)) {
    const int cn = min(SCAN_CHUNK, L - t0);
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int e = tid + j * SCAN_THREADS;
      const int t = e / CPB, cl = e - t * CPB;
      const int c = c0 + cl;
      if (t < cn && c < channels) {
        const size_t n = (size_t)(s0 + t0 + t);
        dt_r[j] = dt_in[n * channels + c] + dt_bias[c];
        x_r[j] = x[n * x_stride + c];
        z_r[j] = z[n * z_stride + c];
      }
    }
#pragma unroll
    for (int j = 0; j < BPT; ++j) {
      const int e = tid + j * SCAN_THREADS;
      const int t = e / NP, i = e - t * NP;
      if (t < cn && i < states) {
        const size_t n = (size_t)(s0 + t0 + t);
        b_r[j] = B[n * bc_stride + i];
        c_r[j] = C[n * bc_stride + i];
      }
    }
  };
  auto stage = [&](int t0) __attribute__((always_inline)) {
    const int cn = min(SCAN_CHUNK, L - t0);
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int e = tid + j * SCAN_THREADS;
      const int t = e / CPB, cl = e - t * CPB;
      if (t < cn) {
        const bool in = c0 + cl < channels;
        s_dt[t][cl] = in ? scan_softplus(dt_r[j]) : 0.f;
        s_x[t][cl] = in ? to_float(x_r[j]) : 0.f;
        s_z[t][cl] = in ? to_float(z_r[j]) : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < BPT; ++j) {
      const int e = tid + j * SCAN_THREADS;
      const int t = e / NP, i = e - t * NP;
      if (t < cn) {
        s_b[t][i] = i < states ? to_float(b_r[j]) : 0.f;
        s_c[t][i] = i < states ? to_float(c_r[j]) : 0.f;
      }
    }
  };
  ask(0);
  for (int t0 = 0; t0 < L; t0 += SCAN_CHUNK) {
    const int cn = min(SCAN_CHUNK, L - t0);
    __syncthreads();    // the chunk before has been walked
    stage(t0);
    __syncthreads();
    if (t0 + SCAN_CHUNK < L) ask(t0 + SCAN_CHUNK);
    // one token: everything but the last multiply-add of a state is independent of the state, so the tokens of a
    // group of four overlap; the exponential is the hardware's 2^x
    auto token = [&](int t) __attribute__((always_inline)) -> float {
      const float dt = s_dt[t][ch_local], xv = s_x[t][ch_local];
      const float dx = dt * xv;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < SPT; ++i) {
        S[i] = fmaf(__builtin_amdgcn_exp2f(dt * a[i]), S[i], dx * s_b[t][part * SPT + i]);
        acc = fmaf(S[i], s_c[t][part * SPT + i], acc);
      }
      return fmaf(dskip, xv, scan_group_sum<LPC>(acc));
    };
    auto gate_store = [&](int t, float y) __attribute__((always_inline)) {
      const float zv = s_z[t][ch_local];
      const float g = sizeof(T) == 4 ? zv / (1.0f + expf(-zv)) : fast_silu(zv);
      out[(size_t)(s0 + t0 + t) * out_stride + ch] = from_float<T>(y * g);
    };
    int t = 0;
    if (LPC >= 4) {
      // four tokens at a time; then lane u of a channel's group gates and stores token u, so that the gate's
      // arithmetic runs once for the four tokens and not once for each
      for (; t + 4 <= cn; t += 4) {
        const float y0 = token(t), y1 = token(t + 1), y2 = token(t + 2), y3 = token(t + 3);
        const int u = part & 3;
        const float y = u == 0 ? y0 : (u == 1 ? y1 : (u == 2 ? y2 : y3));
        if (live && part < 4) gate_store(t + u, y);
      }
    }
    for (; t < cn; ++t) {
      const float y = token(t);
      if (live && part == 0) gate_store(t, y);
    }
  }
#pragma unroll
  for (int i = 0; i < SPT; ++i) {
    const int n = part * SPT + i;
    if (live && n < states) Sg[n] = S[i];
  }
}

}  // namespace

// x [n, channels] (row stride x_stride), z alike, B and C [n, states] (row stride bc_stride) in `dtype`; dt_in float
// [n, channels] (the step size before its bias and softplus); A float [channels, states] (negative); state float
// [slots, channels, states]; out [n, channels] in `dtype`.
extern "C" int ms_selective_scan(const void* x, long long x_stride, const float* dt_in, const float* dt_bias, const float* A,
                                 const void* B, const void* C, long long bc_stride, const float* D, const void* z,
                                 long long z_stride, float* state, const int* q_start, const int* state_slots, void* out,
                                 long long out_stride, int n_requests, int channels, int states, int dtype,
                                 hipStream_t stream) {
  if (n_requests <= 0) return MS_OK;
  if (channels <= 0 || states <= 0) return MS_BAD_ARG;
  if (states > 256 || n_requests > 65535) return MS_UNSUPPORTED;
  int spt, lpc;
  if (states <= 4) { spt = 4; lpc = 1; }
  else if (states <= 8) { spt = 4; lpc = 2; }
  else if (states <= 16) { spt = 4; lpc = 4; }
  else if (states <= 32) { spt = 4; lpc = 8; }
  else if (states <= 64) { spt = 4; lpc = 16; }
  else if (states <= 128) { spt = 8; lpc = 16; }
  else { spt = 16; lpc = 16; }
  const int cpb = SCAN_THREADS / lpc;
  dim3 grid((channels + cpb - 1) / cpb, n_requests), block(SCAN_THREADS);
#define LAUNCH(T, SPT, LPC)                                                                                           \
  selective_scan_kernel<T, SPT, LPC><<<grid, block, 0, stream>>>(                                                     \
      (const T*)x, (size_t)x_stride, dt_in, dt_bias, A, (const T*)B, (const T*)C, (size_t)bc_stride, D, (const T*)z,  \
      (size_t)z_stride, state, q_start, state_slots, (T*)out, (size_t)out_stride, channels, states)
#define BY_SHAPE(T)                                                                                                   \
  do {                                                                                                                \
    if (lpc == 1) LAUNCH(T, 4, 1);                                                                                    \
    else if (lpc == 2) LAUNCH(T, 4, 2);                                                                               \
    else if (lpc == 4) LAUNCH(T, 4, 4);                                                                               \
    else if (lpc == 8) LAUNCH(T, 4, 8);                                                                               \
    else if (spt == 4) LAUNCH(T, 4, 16);                                                                              \
    else if (spt == 8) LAUNCH(T, 8, 16);                                                                              \
    else LAUNCH(T, 16, 16);                                                                                           \
  } while (0)
  if (dtype == MS_F32) BY_SHAPE(float);
  else if (dtype == MS_BF16) BY_SHAPE(bf16);
  else return MS_BAD_ARG;
#undef BY_SHAPE
#undef LAUNCH
  return ms_launch_status();
}
