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
  hipLaunchKernelGGL(conv_silu_kernel, dim3(T_, by), dim3(256), 0, stream, in, in_stride, in_off, w, bias, carry,
                     carry_stride, token_entry, q_start, entry_slot, out, channels, taps);
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


// The same recurrence with the state in registers, for shapes where a thread's share of a column fits there
// (state rows <= SCAN_NPT * (256 / PC)).  One block per (entry, head, slice of PC columns of the head): thread
// (r, p) owns rows n = r, r + R, ... of column p.  The entry's tokens are walked in chunks of up to SCAN_CHUNK: a chunk's
// x, B, C, step sizes and decays are staged in shared memory (the next chunk's loads are issued before the
// current chunk is worked on and land in the other buffer), every thread moves its rows through the chunk's
// tokens, leaving one partial sum per token, and after one barrier the block adds each token's R partial sums in
// the order of r.  A token's result does not depend on where the chunks or the entries are cut: the operations
// on a state element and their order are the same.
#define SCAN_NPT 16
#define SCAN_CHUNK 16
__global__ void __launch_bounds__(SCAN_THREADS)
ssm_scan_reg_kernel(const float* __restrict__ xbc, const float* __restrict__ proj, int proj_stride, int dt_off,
                    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                    float* __restrict__ state, long long state_stride, long long state_off,
                    const int* __restrict__ q_start, const int* __restrict__ entry_slot, float* __restrict__ y,
                    int heads, int groups, int N, int P, int PC, int chunk, int write_state) {
  extern __shared__ float shared[];
  const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * PC, g = h / (heads / groups);
  const int R = SCAN_THREADS / PC;
  const int tid = threadIdx.x;
  const bool active = tid < R * PC;
  const int p = tid % PC, r = tid / PC;
  const int per_buf = chunk * (2 * N + PC + 2);          // B | C | x | dt | decay of one chunk
  float* part = shared + 2 * per_buf;                     // [chunk][R][PC]
  const int channels = heads * P + 2 * groups * N;
  const int first = q_start[b], end = q_start[b + 1];
  float* row = state + (size_t)entry_slot[b] * state_stride + state_off + (size_t)h * N * P + p0;
  float s[SCAN_NPT];
#pragma unroll
  for (int k = 0; k < SCAN_NPT; ++k) {
    const int n = r + k * R;
    s[k] = (active && n < N) ? row[(size_t)n * P + p] : 0.f;
  }
  const float neg_rate = -expf(a_log[h]);
  const float bias = dt_bias[h], skip = d_skip[h];
  const int per_chunk = chunk * (2 * N + PC);             // staged values of a chunk (B, C, x), then chunk step sizes
  constexpr int STAGE = 20;                                // values a thread stages per chunk, at most
  // stage(c0, buf): tokens c0 .. c0+chunk-1 of the entry into buffer buf
  auto fetch = [&](int c0, float (&v)[STAGE]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < STAGE; ++u) {
      const int e = tid + u * SCAN_THREADS;
      float val = 0.f;
      if (e < per_chunk) {
        const int t = e / (2 * N + PC), j = e % (2 * N + PC);
        if (c0 + t < end) {
          const float* in = xbc + (size_t)(c0 + t) * channels;
          val = j < N ? in[heads * P + g * N + j]
                      : (j < 2 * N ? in[heads * P + groups * N + g * N + (j - N)] : in[h * P + p0 + (j - 2 * N)]);
        }
      } else if (e < per_chunk + chunk) {
        const int t = e - per_chunk;
        val = c0 + t < end ? proj[(size_t)(c0 + t) * proj_stride + dt_off + h] : 0.f;
      }
      v[u] = val;
    }
  };
  auto put = [&](const float (&v)[STAGE], float* buf) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < STAGE; ++u) {
      const int e = tid + u * SCAN_THREADS;
      if (e < per_chunk) {
        const int t = e / (2 * N + PC), j = e % (2 * N + PC);
        buf[t * (2 * N + PC) + j] = v[u];
      } else if (e < per_chunk + chunk) {
        const int t = e - per_chunk;
        const float raw = v[u] + bias;
        const float dt = raw > 0.f ? raw + log1pf(expf(-raw)) : log1pf(expf(raw));
        buf[per_chunk + t] = dt;
        buf[per_chunk + chunk + t] = expf(neg_rate * dt);
      }
    }
  };
  float v[STAGE];
  fetch(first, v);
  put(v, shared);
  __syncthreads();
  int turn = 0;
  for (int c0 = first; c0 < end; c0 += chunk) {
    float* buf = shared + turn * per_buf;
    const bool more = c0 + chunk < end;
    if (more) fetch(c0 + chunk, v);
    const int n_tok = end - c0 < chunk ? end - c0 : chunk;
    if (active) {
      for (int t = 0; t < n_tok; ++t) {
        const float* bs = buf + t * (2 * N + PC);
        const float* cs = bs + N;
        const float dtx = buf[per_chunk + t] * bs[2 * N + p];
        const float a = buf[per_chunk + chunk + t];
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < SCAN_NPT; ++k) {
          const int n = r + k * R;
          if (n < N) {
            s[k] = a * s[k] + bs[n] * dtx;
            acc += s[k] * cs[n];
          }
        }
        part[(t * R + r) * PC + p] = acc;
      }
    }
    __syncthreads();
    for (int e = tid; e < n_tok * PC; e += SCAN_THREADS) {
      const int t = e / PC, pp = e % PC;
      float sum = 0.f;
      for (int k = 0; k < R; ++k) sum += part[(t * R + k) * PC + pp];
      y[(size_t)(c0 + t) * heads * P + h * P + p0 + pp] = sum + skip * buf[t * (2 * N + PC) + 2 * N + pp];
    }
    if (more) put(v, shared + (1 - turn) * per_buf);
    __syncthreads();
    turn = 1 - turn;
  }
  if (write_state && active) {
#pragma unroll
    for (int k = 0; k < SCAN_NPT; ++k) {
      const int n = r + k * R;
      if (n < N) row[(size_t)n * P + p] = s[k];
    }
  }
}

extern "C" int ullm_ssm_scan(const float* xbc, const float* proj, int proj_stride, int dt_off, const float* dt_bias,
                             const float* a_log, const float* d_skip, float* state, long long state_stride,
                             long long state_off, const int* q_start, const int* entry_slot, float* y, int B_,
                             int heads, int groups, int N, int P, int write_state, hipStream_t stream) {
  if (B_ <= 0) return 0;
  if (heads <= 0 || groups <= 0 || heads % groups || N <= 0 || P <= 0 || P > SCAN_THREADS) return ULLM_ERR_SHAPE;
  // columns of a head per block: 16 where the head cuts into such slices, else the whole head
  const int PC = P % 16 == 0 ? 16 : P;
  const int R_reg = SCAN_THREADS / PC;
  if ((N + R_reg - 1) / R_reg <= SCAN_NPT) {
    int chunk = SCAN_CHUNK;
    while (chunk > 1 && ((size_t)chunk * (2 * N + PC) + chunk > 20 * SCAN_THREADS ||
                         (2 * (size_t)chunk * (2 * N + PC + 2) + (size_t)chunk * R_reg * PC) * sizeof(float) > 64 * 1024))
      chunk /= 2;
    const size_t need = (2 * (size_t)chunk * (2 * N + PC + 2) + (size_t)chunk * R_reg * PC) * sizeof(float);
    if ((size_t)chunk * (2 * N + PC) + chunk <= 20 * SCAN_THREADS && need <= 64 * 1024) {
      hipLaunchKernelGGL(ssm_scan_reg_kernel, dim3(B_, heads, P / PC), dim3(SCAN_THREADS), need, stream, xbc, proj,
                         proj_stride, dt_off, dt_bias, a_log, d_skip, state, state_stride, state_off, q_start, entry_slot,
                         y, heads, groups, N, P, PC, chunk, write_state);
      ULLM_LAUNCH_CHECK();
    }
  }
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

extern "C" int ullm_gated_group_norm(const float* y, const float* proj, int proj_stride, int z_off, const float* gain,
                                     float eps, void* out, int T_, int width, int parts, int out_dtype,
                                     hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (width <= 0 || parts <= 0 || width % parts || parts > 65535) return ULLM_ERR_SHAPE;
  const int part = width / parts;
#define GO(TY) hipLaunchKernelGGL(gated_group_norm_kernel<TY>, dim3(T_, parts), dim3(256), 0, stream, y, proj, \
    proj_stride, z_off, gain, eps, (TY*)out, width, part)
  if (out_dtype == ULLM_F32) GO(float);
  else if (out_dtype == ULLM_BF16) GO(bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}
