// Kernels of recurrent mixers with a fixed-size state per request: a short causal convolution per
// channel whose last inputs are carried from step to step, the selective state-space recurrence
// (one matrix state per head, decayed and updated token by token), and the gated, grouped RMS norm
// behind it.  Everything here is 32-bit: inputs are float32 rows of the input projection, the state
// rows are float32, sums have a fixed order that depends on the token alone.  A batch is any mix of
// prompt portions and single tokens: entry b owns tokens q_start[b] .. q_start[b+1]-1 and the state
// row entry_slot[b]; the rows of requests that start at their first token are zero when a step begins.
#include "common.h"

#define CONV_MAX_TAPS 16

__device__ __forceinline__ float silu_f32(float z) { return z / (1.f + expf(-z)); }

// ------------------------------------------------------------------ causal convolution + silu
// out[t, c] = silu(bias[c] + sum_j w[c, j] * in(i - (taps-1) + j)) for the token's index i inside its
// entry, where in(l) is this step's input row q_start[b] + l for l >= 0 and otherwise what the state row
// holds: carry[slot, (l + taps-1) * channels + c], the inputs of the taps-1 tokens before the step.
__global__ void __launch_bounds__(256)
conv_silu_kernel(const float* __restrict__ in, int in_stride, int in_off, const float* __restrict__ w,
                 const float* __restrict__ bias, const float* __restrict__ carry, long long carry_stride,
                 const int* __restrict__ token_entry, const int* __restrict__ q_start,
                 const int* __restrict__ entry_slot, float* __restrict__ out, int channels, int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int b = token_entry[t];
  const int first = q_start[b];
  const int i = t - first;
  const float* old = carry + (size_t)entry_slot[b] * carry_stride;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int l = i - (taps - 1) + j;
    const float v = l >= 0 ? in[(size_t)(first + l) * in_stride + in_off + c] : old[(size_t)(l + taps - 1) * channels + c];
    acc += w[(size_t)c * taps + j] * v;
  }
  out[(size_t)t * channels + c] = silu_f32(acc);
}

// The same, four neighbouring channels a thread (16-byte loads and stores) and ``tok`` tokens a block, for rows
// and offsets that are multiples of four values.  A channel's sum has the same terms in the same order.
typedef __attribute__((ext_vector_type(4))) float conv_f32x4;
template <int TAPS>
__global__ void __launch_bounds__(256)
conv_silu_vec_kernel(const float* __restrict__ in, int in_stride, int in_off, const float* __restrict__ w,
                     const float* __restrict__ bias, const float* __restrict__ carry, long long carry_stride,
                     const int* __restrict__ token_entry, const int* __restrict__ q_start,
                     const int* __restrict__ entry_slot, float* __restrict__ out, int T_, int channels, int tok) {
  const int c = 4 * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c >= channels) return;
  float wv[4][TAPS];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wv[q][j] = w[(size_t)(c + q) * TAPS + j];
  const conv_f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const conv_f32x4 b4 = bias ? *reinterpret_cast<const conv_f32x4*>(bias + c) : zero4;
  const int t0 = blockIdx.x * tok;
  for (int t = t0; t < t0 + tok && t < T_; ++t) {
    const int b = token_entry[t];
    const int first = q_start[b];
    const int i = t - first;
    const float* old = carry + (size_t)entry_slot[b] * carry_stride;
    conv_f32x4 acc = b4;
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int l = i - (TAPS - 1) + j;
      const float* src = l >= 0 ? in + (size_t)(first + l) * in_stride + in_off + c : old + (size_t)(l + TAPS - 1) * channels + c;
      const conv_f32x4 v = *reinterpret_cast<const conv_f32x4*>(src);
      acc.x += wv[0][j] * v.x;
      acc.y += wv[1][j] * v.y;
      acc.z += wv[2][j] * v.z;
      acc.w += wv[3][j] * v.w;
    }
    const conv_f32x4 r = {silu_f32(acc.x), silu_f32(acc.y), silu_f32(acc.z), silu_f32(acc.w)};
    *reinterpret_cast<conv_f32x4*>(out + (size_t)t * channels + c) = r;
  }
}

// After the convolution: the state row takes the inputs of the entry's last taps-1 tokens (older ones
// move up where the entry brought fewer).  A thread reads everything it needs before it writes.
__global__ void __launch_bounds__(256)
conv_carry_kernel(const float* __restrict__ in, int in_stride, int in_off, float* __restrict__ carry,
                  long long carry_stride, const int* __restrict__ q_start, const int* __restrict__ entry_slot,
                  int channels, int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[b], n = q_start[b + 1] - first;
  float* row = carry + (size_t)entry_slot[b] * carry_stride;
  float keep[CONV_MAX_TAPS];
#pragma unroll
  for (int k = 0; k < CONV_MAX_TAPS; ++k) {
    if (k < taps - 1) {
      const int l = n - (taps - 1) + k;
      keep[k] = l >= 0 ? in[(size_t)(first + l) * in_stride + in_off + c] : row[(size_t)(k + n) * channels + c];
    }
  }
#pragma unroll
  for (int k = 0; k < CONV_MAX_TAPS; ++k)
    if (k < taps - 1) row[(size_t)k * channels + c] = keep[k];
}

extern "C" int ullm_conv_silu(const float* in, int in_stride, int in_off, const float* w, const float* bias,
                              float* carry, long long carry_stride, const int* token_entry, const int* q_start,
                              const int* entry_slot, float* out, int T_, int B_, int channels, int taps,
                              int update_carry, hipStream_t stream) {
  if (T_ <= 0 || B_ <= 0) return 0;
  if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS || in_stride < in_off + channels) return ULLM_ERR_SHAPE;
  const int by = (channels + 255) / 256;
  const bool by16 = channels % 4 == 0 && in_stride % 4 == 0 && in_off % 4 == 0 && carry_stride % 4 == 0 &&
                    ((uintptr_t)in | (uintptr_t)carry | (uintptr_t)out | (uintptr_t)bias) % 16 == 0;
  if (by16 && taps >= 2 && taps <= 4) {
    // a block walks several tokens where the step has many (the weights are read once a thread)
    const int tok = T_ >= 1024 ? 8 : (T_ >= 256 ? 2 : 1);
    const dim3 grid((T_ + tok - 1) / tok, (channels / 4 + 255) / 256);
#define CONV_GO(TAPS) hipLaunchKernelGGL(conv_silu_vec_kernel<TAPS>, grid, dim3(256), 0, stream, in, in_stride, in_off, w, \
    bias, carry, carry_stride, token_entry, q_start, entry_slot, out, T_, channels, tok)
    if (taps == 2) CONV_GO(2);
    else if (taps == 3) CONV_GO(3);
    else CONV_GO(4);
#undef CONV_GO
  } else {
    hipLaunchKernelGGL(conv_silu_kernel, dim3(T_, by), dim3(256), 0, stream, in, in_stride, in_off, w, bias, carry,
                       carry_stride, token_entry, q_start, entry_slot, out, channels, taps);
  }
  if (update_carry && taps > 1)
    hipLaunchKernelGGL(conv_carry_kernel, dim3(B_, by), dim3(256), 0, stream, in, in_stride, in_off, carry, carry_stride,
                       q_start, entry_slot, channels, taps);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ selective state-space recurrence
// Per head h (group g = h / (heads / groups)) and token, with S [N, P] the head's state:
//   dt = softplus(dt_raw[h] + dt_bias[h]);  a = exp(-exp(a_log[h]) * dt)
//   S = a * S + dt * B_g x_h^T;   y_h = S^T C_g + d_skip[h] * x_h
// x, B, C are columns of ``xbc`` [T, heads*P + 2*groups*N] (x | B | C); dt_raw is column dt_off + h of ``proj``.
// One block per (entry, head): the state lives in shared memory while the block walks the entry's tokens
// in order and goes back to the state row at the end.  Thread (r, p) owns rows n = r, r + R, ... of column p;
// a token's output sums the R partial sums in the order of r.
#define SCAN_THREADS 256
__global__ void __launch_bounds__(SCAN_THREADS)
ssm_scan_kernel(const float* __restrict__ xbc, const float* __restrict__ proj, int proj_stride, int dt_off,
                const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                float* __restrict__ state, long long state_stride, long long state_off,
                const int* __restrict__ q_start, const int* __restrict__ entry_slot, float* __restrict__ y,
                int heads, int groups, int N, int P, int PP, int write_state) {
  extern __shared__ float shared[];
  const int b = blockIdx.x, h = blockIdx.y, g = h / (heads / groups);
  const int R = SCAN_THREADS / PP;
  const int p = threadIdx.x % PP, r = threadIdx.x / PP;
  float* S = shared;                    // [N, P]
  float* xs = S + (size_t)N * P;        // [P]
  float* bs = xs + P;                   // [N]  dt * B
  float* cs = bs + N;                   // [N]
  float* part = cs + N;                 // [R, PP]
  const int channels = heads * P + 2 * groups * N;
  const int first = q_start[b], end = q_start[b + 1];
  float* row = state + (size_t)entry_slot[b] * state_stride + state_off + (size_t)h * N * P;
  for (int e = threadIdx.x; e < N * P; e += SCAN_THREADS) S[e] = row[e];
  const float neg_rate = -expf(a_log[h]);
  const float bias = dt_bias[h], skip = d_skip[h];
  for (int t = first; t < end; ++t) {
    const float raw = proj[(size_t)t * proj_stride + dt_off + h] + bias;
    // softplus without a clamp: log(1 + e^raw), written so that neither side overflows
    const float dt = raw > 0.f ? raw + log1pf(expf(-raw)) : log1pf(expf(raw));
    const float a = expf(neg_rate * dt);
    const float* in = xbc + (size_t)t * channels;
    __syncthreads();                    // the token before is done with xs, bs, cs, part (and S is loaded)
    for (int e = threadIdx.x; e < P; e += SCAN_THREADS) xs[e] = in[h * P + e];
    for (int e = threadIdx.x; e < N; e += SCAN_THREADS) {
      bs[e] = dt * in[heads * P + g * N + e];
      cs[e] = in[heads * P + groups * N + g * N + e];
    }
    __syncthreads();
    float acc = 0.f;
    if (p < P) {
      const float x = xs[p];
      for (int n = r; n < N; n += R) {
        const float s = a * S[n * P + p] + bs[n] * x;
        S[n * P + p] = s;
        acc += s * cs[n];
      }
    }
    part[r * PP + p] = acc;
    __syncthreads();
    if (threadIdx.x < P) {
      float sum = 0.f;
      for (int k = 0; k < R; ++k) sum += part[k * PP + threadIdx.x];
      y[(size_t)t * heads * P + h * P + threadIdx.x] = sum + skip * xs[threadIdx.x];
    }
  }
  __syncthreads();
  if (write_state)
    for (int e = threadIdx.x; e < N * P; e += SCAN_THREADS) row[e] = S[e];
}


// The same recurrence with the state in registers.  One block per (entry, head, slice of PC columns of the head):
// thread (r, p) owns the NPT rows n = r * NPT .. of column p, R = 256 / PC such threads cover R * NPT >= N rows (rows
// from N on are zero: their B and C are staged as zeros, so the inner loop has no bounds).  The entry's tokens are
// walked in chunks of SCAN_CHUNK: 16 lanes share a token and bring its B, C and x as 16-byte loads, the chunk's
// step sizes and decays are worked out once, all of it staged in shared memory (the next chunk's loads are issued
// before the current chunk is worked on and land in the other buffer); every thread moves its rows through the
// chunk's tokens with 16-byte reads of B and C, leaving one partial sum per token, and after one barrier the block
// adds each token's R partial sums in the order of r.  Tokens past the entry's end are staged with a step size of
// zero (decay 1, nothing added), so the token loop runs in fours without a tail.  A token's result does not depend
// on where the chunks or the entries are cut: the operations on a state element and their order are the same.
#define SCAN_CHUNK 16
typedef __attribute__((ext_vector_type(4))) float scan_f32x4;

// A barrier for shared memory alone: the block's accesses to shared memory are complete, while loads and stores of
// global memory stay in flight (the barrier of __syncthreads also waits for those: the next chunk's loads and the
// results' stores would be waited for twice a chunk).
__device__ __forceinline__ void shared_memory_barrier() {
#ifdef __HIP_DEVICE_COMPILE__
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#endif
}

template <int PC, int NPT>
__global__ void __launch_bounds__(SCAN_THREADS)
ssm_scan_tile_kernel(const float* __restrict__ xbc, const float* __restrict__ proj, int proj_stride, int dt_off,
                     const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                     float* __restrict__ state, long long state_stride, long long state_off,
                     const int* __restrict__ q_start, const int* __restrict__ entry_slot, float* __restrict__ y,
                     int heads, int groups, int N, int P, int write_state) {
  constexpr int R = SCAN_THREADS / PC;              // threads that share a column
  constexpr int NP = R * NPT;                       // state rows the block covers
  constexpr int NB4 = (NP / 4 + 15) / 16;           // 16-byte loads of B (and of C) per lane and chunk
  constexpr int XL = PC / 4;                        // lanes of a token's 16 that bring x
  constexpr int ROW = 2 * NP + PC;                  // staged values of a token: B | C | x
  constexpr int PER_BUF = SCAN_CHUNK * ROW + 2 * SCAN_CHUNK;   // ... then the chunk's step sizes and decays
  static_assert(PC % 4 == 0 && PC <= 64 && NP % 4 == 0, "slices are cut in 16-byte pieces");
  extern __shared__ __attribute__((aligned(16))) float shared[];
  float* part = shared + 2 * PER_BUF;               // [chunk][R][PC]
  const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * PC, g = h / (heads / groups);
  const int tid = threadIdx.x;
  const int p = tid % PC, r = tid / PC;
  const bool column = p0 + p < P;
  const int channels = heads * P + 2 * groups * N;
  const int first = q_start[b], end = q_start[b + 1];
  float* row = state + (size_t)entry_slot[b] * state_stride + state_off + (size_t)h * N * P + p0;
  float s[NPT];
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int n = r * NPT + k;
    s[k] = (column && n < N) ? row[(size_t)n * P + p] : 0.f;
  }
  const float neg_rate = -expf(a_log[h]);
  const float bias = dt_bias[h], skip = d_skip[h];
  const int tl = tid / 16, ln = tid % 16;            // staging: token of the chunk, lane of its 16
  const float* b_col = xbc + (size_t)heads * P + (size_t)g * N;
  const float* c_col = b_col + (size_t)groups * N;
  const float* x_col = xbc + (size_t)h * P + p0;
  const scan_f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  scan_f32x4 vb[NB4], vc[NB4], vx;
  float vdt;
  auto fetch = [&](int c0) __attribute__((always_inline)) {
    const int tok = c0 + tl;
    const bool live = tok < end;
    const size_t base = (size_t)tok * channels;
#pragma unroll
    for (int u = 0; u < NB4; ++u) {
      const int n = 4 * (ln + 16 * u);
      const bool in = live && n < N;
      vb[u] = in ? *reinterpret_cast<const scan_f32x4*>(b_col + base + n) : zero4;
      vc[u] = in ? *reinterpret_cast<const scan_f32x4*>(c_col + base + n) : zero4;
    }
    vx = (live && ln < XL && p0 + 4 * ln < P) ? *reinterpret_cast<const scan_f32x4*>(x_col + base + 4 * ln) : zero4;
    vdt = (live && ln == 15) ? proj[(size_t)tok * proj_stride + dt_off + h] : 0.f;
  };
  auto put = [&](int c0, float* buf) __attribute__((always_inline)) {
    float* dst = buf + tl * ROW;
#pragma unroll
    for (int u = 0; u < NB4; ++u) {
      const int n = 4 * (ln + 16 * u);
      if (n < NP) {
        *reinterpret_cast<scan_f32x4*>(dst + n) = vb[u];
        *reinterpret_cast<scan_f32x4*>(dst + NP + n) = vc[u];
      }
    }
    if (ln < XL) *reinterpret_cast<scan_f32x4*>(dst + 2 * NP + 4 * ln) = vx;
    if (ln == 15) {
      float dt = 0.f, a = 1.f;
      if (c0 + tl < end) {
        // softplus without a clamp: max(raw, 0) + log(1 + e^-|raw|), one exponential and one logarithm;
        // log(u) * e / (u - 1) with u = 1 + e rounded is log(1 + e) to a few units in the last place for any e
        // (every wave has such lanes, so whatever stands here is issued by all of them once a chunk)
        const float raw = vdt + bias;
        const float e = expf(-fabsf(raw)), u = 1.f + e;
        const float l = u == 1.f ? e : logf(u) * (e / (u - 1.f));
        dt = fmaxf(raw, 0.f) + l;
        a = expf(neg_rate * dt);
      }
      buf[SCAN_CHUNK * ROW + tl] = dt;
      buf[SCAN_CHUNK * ROW + SCAN_CHUNK + tl] = a;
    }
  };
  struct TokenIn {
    float b[NPT], c[NPT];
    float dtx, a;
  };
  auto read_token = [&](const float* buf, int t, TokenIn& in) __attribute__((always_inline)) {
    const float* bs = buf + t * ROW + r * NPT;
    if constexpr (NPT % 4 == 0) {
#pragma unroll
      for (int k = 0; k < NPT; k += 4) {
        const scan_f32x4 bb = *reinterpret_cast<const scan_f32x4*>(bs + k);
        const scan_f32x4 cc = *reinterpret_cast<const scan_f32x4*>(bs + NP + k);
        in.b[k] = bb.x, in.b[k + 1] = bb.y, in.b[k + 2] = bb.z, in.b[k + 3] = bb.w;
        in.c[k] = cc.x, in.c[k + 1] = cc.y, in.c[k + 2] = cc.z, in.c[k + 3] = cc.w;
      }
    } else {
#pragma unroll
      for (int k = 0; k < NPT; ++k) in.b[k] = bs[k], in.c[k] = bs[NP + k];
    }
    in.dtx = buf[SCAN_CHUNK * ROW + t] * buf[t * ROW + 2 * NP + p];
    in.a = buf[SCAN_CHUNK * ROW + SCAN_CHUNK + t];
  };
  // one token: every row of this thread decays and takes its share of B x; returns the thread's part of y
  auto move_rows = [&](const TokenIn& in) __attribute__((always_inline)) {
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < NPT; ++k) {
      s[k] = in.a * s[k] + in.b[k] * in.dtx;
      acc += s[k] * in.c[k];
    }
    return acc;
  };
  fetch(first);
  put(first, shared);
  shared_memory_barrier();
  int turn = 0;
  for (int c0 = first; c0 < end; c0 += SCAN_CHUNK) {
    const float* buf = shared + turn * PER_BUF;
    const bool more = c0 + SCAN_CHUNK < end;
    if (more) fetch(c0 + SCAN_CHUNK);
    const int n_tok = end - c0 < SCAN_CHUNK ? end - c0 : SCAN_CHUNK;
    const int t_end = (n_tok + 3) & ~3;
    // a token's B, C, x, step size and decay are read one token ahead of the arithmetic that uses them, into two
    // sets of registers that take turns: the reads' latency passes while the token before is worked on
    TokenIn in_a, in_b;
    read_token(buf, 0, in_a);
    for (int t = 0; t < t_end; t += 2) {
      read_token(buf, t + 1, in_b);
      part[(t * R + r) * PC + p] = move_rows(in_a);
      read_token(buf, t + 2 < SCAN_CHUNK ? t + 2 : SCAN_CHUNK - 1, in_a);
      part[((t + 1) * R + r) * PC + p] = move_rows(in_b);
    }
    shared_memory_barrier();
    for (int e = tid; e < n_tok * PC; e += SCAN_THREADS) {
      const int t = e / PC, pp = e % PC;
      if (p0 + pp < P) {
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < R; ++k) sum += part[(t * R + k) * PC + pp];
        y[(size_t)(c0 + t) * heads * P + h * P + p0 + pp] = sum + skip * buf[t * ROW + 2 * NP + pp];
      }
    }
    if (more) put(c0 + SCAN_CHUNK, shared + (1 - turn) * PER_BUF);
    shared_memory_barrier();
    turn = 1 - turn;
  }
  if (write_state && column) {
#pragma unroll
    for (int k = 0; k < NPT; ++k) {
      const int n = r * NPT + k;
      if (n < N) row[(size_t)n * P + p] = s[k];
    }
  }
}

template <int PC, int NPT>
static int launch_scan_tile(const float* xbc, const float* proj, int proj_stride, int dt_off, const float* dt_bias,
                            const float* a_log, const float* d_skip, float* state, long long state_stride,
                            long long state_off, const int* q_start, const int* entry_slot, float* y, int B_, int heads,
                            int groups, int N, int P, int write_state, hipStream_t stream) {
  constexpr int R = SCAN_THREADS / PC, NP = R * NPT;
  constexpr size_t need = (2 * (size_t)(SCAN_CHUNK * (2 * NP + PC) + 2 * SCAN_CHUNK) + (size_t)SCAN_CHUNK * R * PC) * sizeof(float);
  static_assert(need <= 160 * 1024, "a block's staging fits the shared memory of a compute unit");
  if (need > 64 * 1024) {
    const hipError_t e = hipFuncSetAttribute((const void*)ssm_scan_tile_kernel<PC, NPT>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)need);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL((ssm_scan_tile_kernel<PC, NPT>), dim3(B_, heads, (P + PC - 1) / PC), dim3(SCAN_THREADS), need, stream,
                     xbc, proj, proj_stride, dt_off, dt_bias, a_log, d_skip, state, state_stride, state_off, q_start,
                     entry_slot, y, heads, groups, N, P, write_state);
  ULLM_LAUNCH_CHECK();
}

extern "C" int ullm_ssm_scan(const float* xbc, const float* proj, int proj_stride, int dt_off, const float* dt_bias,
                             const float* a_log, const float* d_skip, float* state, long long state_stride,
                             long long state_off, const int* q_start, const int* entry_slot, float* y, int B_,
                             int heads, int groups, int N, int P, int write_state, hipStream_t stream) {
  if (B_ <= 0) return 0;
  if (heads <= 0 || groups <= 0 || heads % groups || N <= 0 || P <= 0 || P > SCAN_THREADS) return ULLM_ERR_SHAPE;
#define SCAN_GO(PC, NPT) return launch_scan_tile<PC, NPT>(xbc, proj, proj_stride, dt_off, dt_bias, a_log, d_skip, state, \
    state_stride, state_off, q_start, entry_slot, y, B_, heads, groups, N, P, write_state, stream)
  if (N % 4 == 0 && P % 4 == 0) {
    // whole rows of 64 columns a block where there are blocks enough without slicing the heads (a step of many
    // requests: the state's rows are then read and written as whole lines); else slices of 16 columns
    if (P % 64 == 0 && N <= 128 && (long long)B_ * heads >= 1024) {
      if (N <= 32) SCAN_GO(64, 8);
      if (N <= 64) SCAN_GO(64, 16);
      SCAN_GO(64, 32);
    }
    if (N <= 16) SCAN_GO(16, 1);
    if (N <= 32) SCAN_GO(16, 2);
    if (N <= 64) SCAN_GO(16, 4);
    if (N <= 128) SCAN_GO(16, 8);
    if (N <= 256) SCAN_GO(16, 16);
  }
#undef SCAN_GO
  int PP = 1;
  while (PP < P) PP *= 2;
  const int R = SCAN_THREADS / PP;
  const size_t shared = ((size_t)N * P + P + 2 * (size_t)N + (size_t)R * PP) * sizeof(float);
  if (shared > 160 * 1024) return ULLM_ERR_SHAPE;
  if (shared > 64 * 1024) {
    const hipError_t e = hipFuncSetAttribute((const void*)ssm_scan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shared);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(ssm_scan_kernel, dim3(B_, heads), dim3(SCAN_THREADS), shared, stream, xbc, proj, proj_stride, dt_off,
                     dt_bias, a_log, d_skip, state, state_stride, state_off, q_start, entry_slot, y, heads, groups, N, P,
                     PP, write_state);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ gate, then RMS norm in equal parts
// v = y * silu(z) with z = proj[t, z_off + c]; the row is cut into ``parts`` equal parts, each divided by its
// own root mean square (eps inside the root) and multiplied by the gain.  One block per (token, part).
template <typename TY>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ proj, int proj_stride, int z_off,
                        const float* __restrict__ gain, float eps, TY* __restrict__ out, int width, int part) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, k = blockIdx.y;
  const float* yr = y + (size_t)t * width + (size_t)k * part;
  const float* zr = proj + (size_t)t * proj_stride + z_off + (size_t)k * part;
  float ss = 0.f;
  for (int c = threadIdx.x; c < part; c += blockDim.x) {
    const float v = yr[c] * silu_f32(zr[c]);
    ss += v * v;
  }
  const float rs = 1.f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
  TY* o = out + (size_t)t * width + (size_t)k * part;
  const float* gn = gain + (size_t)k * part;
  for (int c = threadIdx.x; c < part; c += blockDim.x) st_f32(o + c, ((yr[c] * silu_f32(zr[c])) * rs) * gn[c]);
}

// The same with one wave per (token, part) and the part's values kept in registers between the sum of squares and
// the scaling (parts of up to 64 * 4 * GN_V values that cut into 16-byte pieces): no barrier, one pass over y and z.
#define GN_V 8
typedef __attribute__((ext_vector_type(4))) float gn_f32x4;
template <typename TY>
__global__ void __launch_bounds__(256)
gated_group_norm_wave_kernel(const float* __restrict__ y, const float* __restrict__ proj, int proj_stride, int z_off,
                             const float* __restrict__ gain, float eps, TY* __restrict__ out, int width, int part,
                             int parts, long long pairs) {
  const long long pair = (long long)blockIdx.x * 4 + threadIdx.x / WAVE;
  if (pair >= pairs) return;
  const int lane = threadIdx.x % WAVE;
  const long long t = pair / parts;
  const int k = (int)(pair % parts);
  const float* yr = y + (size_t)t * width + (size_t)k * part;
  const float* zr = proj + (size_t)t * proj_stride + z_off + (size_t)k * part;
  gn_f32x4 v[GN_V];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < GN_V; ++u) {
    const int c = 4 * (lane + WAVE * u);
    if (c < part) {
      const gn_f32x4 a = *reinterpret_cast<const gn_f32x4*>(yr + c);
      const gn_f32x4 z = *reinterpret_cast<const gn_f32x4*>(zr + c);
      v[u].x = a.x * silu_f32(z.x);
      v[u].y = a.y * silu_f32(z.y);
      v[u].z = a.z * silu_f32(z.z);
      v[u].w = a.w * silu_f32(z.w);
      ss += v[u].x * v[u].x + v[u].y * v[u].y + v[u].z * v[u].z + v[u].w * v[u].w;
    }
  }
  const float rs = 1.f / sqrtf(wave_sum(ss) / (float)part + eps);
  TY* o = out + (size_t)t * width + (size_t)k * part;
  const float* gn = gain + (size_t)k * part;
#pragma unroll
  for (int u = 0; u < GN_V; ++u) {
    const int c = 4 * (lane + WAVE * u);
    if (c < part) {
      const gn_f32x4 g4 = *reinterpret_cast<const gn_f32x4*>(gn + c);
      st_f32(o + c, (v[u].x * rs) * g4.x);
      st_f32(o + c + 1, (v[u].y * rs) * g4.y);
      st_f32(o + c + 2, (v[u].z * rs) * g4.z);
      st_f32(o + c + 3, (v[u].w * rs) * g4.w);
    }
  }
}

extern "C" int ullm_gated_group_norm(const float* y, const float* proj, int proj_stride, int z_off, const float* gain,
                                     float eps, void* out, int T_, int width, int parts, int out_dtype,
                                     hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (width <= 0 || parts <= 0 || width % parts || parts > 65535) return ULLM_ERR_SHAPE;
  const int part = width / parts;
  if (part % 4 == 0 && part <= 64 * 4 * GN_V && proj_stride % 4 == 0 && z_off % 4 == 0 &&
      ((uintptr_t)y | (uintptr_t)proj | (uintptr_t)gain) % 16 == 0) {
    const long long pairs = (long long)T_ * parts;
    const dim3 grid((unsigned)((pairs + 3) / 4));
#define GW(TY) hipLaunchKernelGGL(gated_group_norm_wave_kernel<TY>, grid, dim3(256), 0, stream, y, proj, proj_stride, \
    z_off, gain, eps, (TY*)out, width, part, parts, pairs)
    if (out_dtype == ULLM_F32) GW(float);
    else if (out_dtype == ULLM_BF16) GW(bf16_t);
    else return ULLM_ERR_DTYPE;
#undef GW
    ULLM_LAUNCH_CHECK();
  }
#define GO(TY) hipLaunchKernelGGL(gated_group_norm_kernel<TY>, dim3(T_, parts), dim3(256), 0, stream, y, proj, \
    proj_stride, z_off, gain, eps, (TY*)out, width, part)
  if (out_dtype == ULLM_F32) GO(float);
  else if (out_dtype == ULLM_BF16) GO(bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}
