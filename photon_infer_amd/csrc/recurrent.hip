// Mixers whose memory is a state of fixed size per request: the short causal convolution in
// front of them, the state-space recurrence (Mamba-2 form), the gated delta rule with one decay
// per head and key channel, and the norms behind them.  Everything that enters a recurrence is
// float32 in both compute modes: inputs after the convolution, step sizes, decays, gates, the
// state.  A request's state row lies at state[slots[r]]; a step runs the tokens
// q_start[r] .. q_start[r+1]-1 of request r from that row and leaves the row ready for the next
// step, so a prompt may be cut anywhere.  All sizes are run-time values.
#include "common.h"

#define PI_CONV_MAX_TAPS 8
#define PI_CONV_SEGMENT 64
#define PI_SCAN_COLUMNS 16      // value columns of a wave
#define PI_SCAN_CHUNK 8         // tokens staged through LDS at a time

__device__ inline float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ inline float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ inline float softplus_f(float v) { return v > 20.0f ? v : log1pf(expf(v)); }

// ------------------------------------------------------------------ causal convolution + silu
// out[t, c] = silu(bias[c] + sum_j w[c, j] * u[t - (taps - 1) + j, c]), the last column of w on the
// token itself; inputs before the step's first token come from the request's state (the last
// taps - 1 inputs of earlier steps, zeros at the start of a sequence), which is brought up to
// date here.  A thread owns a channel of one segment of a request's tokens; the thread of the
// first segment reads the old state before it writes the new one, and nobody else touches it.
template <typename TW>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    float* __restrict__ out, long out_stride, const float* __restrict__ in, long in_stride, const TW* __restrict__ w,
    const TW* __restrict__ bias, int C, int taps, const int* __restrict__ q_start, const int* __restrict__ slots,
    float* __restrict__ state, long state_stride) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r = blockIdx.y, seg = blockIdx.z;
  const int qs = q_start[r], n = q_start[r + 1] - qs;
  const int t0 = seg * PI_CONV_SEGMENT;
  if (t0 >= n) return;
  const int t1 = t0 + PI_CONV_SEGMENT < n ? t0 + PI_CONV_SEGMENT : n;
  float* st = state + (long)slots[r] * state_stride;      // [(taps - 1), C]
  // weights and window aligned at the end of fixed arrays: unused leading taps weigh zero
  float wr[PI_CONV_MAX_TAPS], win[PI_CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < PI_CONV_MAX_TAPS; ++j) {
    const int tap = j - (PI_CONV_MAX_TAPS - taps);
    wr[j] = tap >= 0 ? to_float(w[(long)c * taps + tap]) : 0.f;
    win[j] = 0.f;
    if (tap >= 0 && tap < taps - 1) {
      const int src = t0 - (taps - 1) + tap;
      win[j] = src >= 0 ? in[(long)(qs + src) * in_stride + c] : st[(long)(taps - 1 + src) * C + c];
    }
  }
  float old[PI_CONV_MAX_TAPS - 1];
  if (seg == 0) {
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS - 1; ++j) old[j] = j < taps - 1 ? st[(long)j * C + c] : 0.f;
  }
  const float b = bias ? to_float(bias[c]) : 0.f;
  for (int t = t0; t < t1; ++t) {
    win[PI_CONV_MAX_TAPS - 1] = in[(long)(qs + t) * in_stride + c];
    float acc = b;
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS; ++j) acc = fmaf(wr[j], win[j], acc);
    out[(long)(qs + t) * out_stride + c] = silu_f(acc);
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS - 1; ++j) win[j] = win[j + 1];
  }
  if (seg == 0) {
#pragma unroll
    for (int j = 0; j < PI_CONV_MAX_TAPS - 1; ++j) {
      if (j < taps - 1) {
        const int src = n - (taps - 1) + j;
        float v;
        if (src >= 0) {
          v = in[(long)(qs + src) * in_stride + c];
        } else {                  // fewer new tokens than the window holds: the old ones move up
          v = 0.f;
#pragma unroll
          for (int o = 0; o < PI_CONV_MAX_TAPS - 1; ++o) v = (o == j + n) ? old[o] : v;
        }
        st[(long)j * C + c] = v;
      }
    }
  }
}

extern "C" int pi_causal_conv_silu(float* out, long out_stride, const float* in, long in_stride, const void* w, const void* bias,
                                   int w_dtype, int C, int taps, const int* q_start, const int* slots, int R, int longest,
                                   float* state, long state_stride, hipStream_t stream) {
  PI_REQUIRE(C > 0 && taps >= 1 && taps <= PI_CONV_MAX_TAPS, "convolution: %d channels with %d taps (at most %d)", C, taps, PI_CONV_MAX_TAPS);
  PI_REQUIRE(R >= 0 && R <= 65535 && longest >= 0, "convolution: bad step shape (%d requests, longest %d)", R, longest);
  PI_REQUIRE(state_stride >= (long)(taps - 1) * C, "convolution: a state row of %ld floats cannot hold %d x %d inputs", state_stride, taps - 1, C);
  if (R == 0 || longest == 0) return 0;
  const int segs = (longest + PI_CONV_SEGMENT - 1) / PI_CONV_SEGMENT;
  PI_REQUIRE(segs <= 65535, "convolution: a request brings too many tokens (%d)", longest);
  const dim3 grid((C + 255) / 256, R, segs), block(256);
  if (w_dtype == PI_F32)
    hipLaunchKernelGGL(causal_conv_silu_kernel<float>, grid, block, 0, stream, out, out_stride, in, in_stride, (const float*)w,
                       (const float*)bias, C, taps, q_start, slots, state, state_stride);
  else if (w_dtype == PI_BF16)
    hipLaunchKernelGGL(causal_conv_silu_kernel<bf16_t>, grid, block, 0, stream, out, out_stride, in, in_stride, (const bf16_t*)w,
                       (const bf16_t*)bias, C, taps, q_start, slots, state, state_stride);
  else
    return pi_fail("convolution: unsupported weight dtype %d", w_dtype);
  return pi_check_launch("causal_conv_silu");
}

// ------------------------------------------------------------------ how a wave holds a state
// A wave owns 16 value columns of one head of one request.  A column's state (one value per
// key channel / state row) is split over four lanes: lane = 4 * column + part, and a lane keeps
// the rows part * NR .. part * NR + NR - 1 in registers.  Rows beyond the real size are zero in
// every staged vector, so they stay zero in the state and the walk needs no tests.
__device__ inline float quad_sum(float v) {
  v += __shfl_xor(v, 1, PI_WAVE);
  v += __shfl_xor(v, 2, PI_WAVE);
  return v;
}

static inline int scan_rows_per_lane(int rows) {
  for (int nr = 4; nr <= 64; nr *= 2)
    if (4 * nr >= rows) return nr;
  return 0;
}

// ------------------------------------------------------------------ state-space recurrence
// Per head h with group g = h / (H / G), state S [N, P] (float32, zero at the start):
//   dt = softplus(dt_raw + dt_bias[h]);  S <- exp(-exp(A_log[h]) * dt) S + dt * B_t x_t^T;
//   y_t = S^T C_t + D[h] x_t
// x, B, C are columns of the convolution's output: x at 0, B at H * P, C at H * P + G * N.
template <int NR>
__global__ __launch_bounds__(PI_WAVE) void state_space_scan_kernel(
    float* __restrict__ y, long y_stride, const float* __restrict__ xbc, long xbc_stride, const float* __restrict__ dt_raw,
    long dt_stride, const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dskip,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ state, long state_stride, int H, int P,
    int N, int G) {
  constexpr int W = 4 * NR;
  __shared__ float sB[PI_SCAN_CHUNK][W], sC[PI_SCAN_CHUNK][W], sx[PI_SCAN_CHUNK][PI_SCAN_COLUMNS], sdt[PI_SCAN_CHUNK], sa[PI_SCAN_CHUNK];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col = blockIdx.z * PI_SCAN_COLUMNS + lane / 4, part = lane % 4;
  const int g = h / (H / G);
  const int qs = q_start[r], n = q_start[r + 1] - qs;
  if (n <= 0) return;
  float* S = state + (long)slots[r] * state_stride + (long)h * N * P;
  const bool live = col < P;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = part * NR + i;
    s[i] = (live && row < N) ? S[(long)row * P + col] : 0.f;
  }
  const float A = expf(A_log[h]), bias = dt_bias[h], skip = Dskip[h];
  const long b_col = (long)H * P + (long)g * N, c_col = b_col + (long)G * N, x_col = (long)h * P + blockIdx.z * PI_SCAN_COLUMNS;
  for (int c0 = 0; c0 < n; c0 += PI_SCAN_CHUNK) {
    const int cn = n - c0 < PI_SCAN_CHUNK ? n - c0 : PI_SCAN_CHUNK;
    __syncthreads();
    for (int i = lane; i < cn * W; i += PI_WAVE) {
      const int tt = i / W, row = i - tt * W;
      const float* src = xbc + (long)(qs + c0 + tt) * xbc_stride;
      sB[tt][row] = row < N ? src[b_col + row] : 0.f;
      sC[tt][row] = row < N ? src[c_col + row] : 0.f;
    }
    for (int i = lane; i < cn * PI_SCAN_COLUMNS; i += PI_WAVE) {
      const int tt = i / PI_SCAN_COLUMNS, cc = i % PI_SCAN_COLUMNS;
      sx[tt][cc] = blockIdx.z * PI_SCAN_COLUMNS + cc < P ? xbc[(long)(qs + c0 + tt) * xbc_stride + x_col + cc] : 0.f;
    }
    if (lane < cn) {
      const float dt = softplus_f(dt_raw[(long)(qs + c0 + lane) * dt_stride + h] + bias);
      sdt[lane] = dt;
      sa[lane] = expf(-A * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < cn; ++tt) {
      const float x = sx[tt][lane / 4], a = sa[tt], dx = sdt[tt] * x;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        s[i] = fmaf(a, s[i], sB[tt][part * NR + i] * dx);
        acc = fmaf(s[i], sC[tt][part * NR + i], acc);
      }
      acc = quad_sum(acc);
      if (live && part == 0) y[(long)(qs + c0 + tt) * y_stride + (long)h * P + col] = fmaf(skip, x, acc);
    }
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = part * NR + i;
    if (live && row < N) S[(long)row * P + col] = s[i];
  }
}

extern "C" int pi_state_space_scan(float* y, long y_stride, const float* xbc, long xbc_stride, const float* dt_raw, long dt_stride,
                                   const float* dt_bias, const float* A_log, const float* Dskip, const int* q_start,
                                   const int* slots, int R, float* state, long state_stride, int H, int P, int N, int G,
                                   hipStream_t stream) {
  PI_REQUIRE(H > 0 && H <= 65535 && P > 0 && N > 0 && G > 0 && H % G == 0, "state space: bad sizes heads=%d vdim=%d state=%d groups=%d", H, P, N, G);
  PI_REQUIRE(R >= 0 && state_stride >= (long)H * N * P, "state space: a state row of %ld floats cannot hold %d x %d x %d", state_stride, H, N, P);
  const int nr = scan_rows_per_lane(N);
  PI_REQUIRE(nr > 0, "state space: a state of %d rows per head is more than 256", N);
  if (R == 0) return 0;
  const dim3 grid(R, H, (P + PI_SCAN_COLUMNS - 1) / PI_SCAN_COLUMNS), block(PI_WAVE);
#define PI_LAUNCH_SS(NR_)                                                                                                     \
  hipLaunchKernelGGL(state_space_scan_kernel<NR_>, grid, block, 0, stream, y, y_stride, xbc, xbc_stride, dt_raw, dt_stride,  \
                     dt_bias, A_log, Dskip, q_start, slots, state, state_stride, H, P, N, G)
  switch (nr) {
    case 4: PI_LAUNCH_SS(4); break;
    case 8: PI_LAUNCH_SS(8); break;
    case 16: PI_LAUNCH_SS(16); break;
    case 32: PI_LAUNCH_SS(32); break;
    default: PI_LAUNCH_SS(64); break;
  }
#undef PI_LAUNCH_SS
  return pi_check_launch("state_space_scan");
}

// ------------------------------------------------------------------ gate, then norm in equal parts
// out[t, i] = mult * w[i] * v[i] / sqrt(mean over i's part of v^2 + eps),  v = y * silu(z).
// One block per (token, part).
template <typename TO>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(TO* __restrict__ out, long out_stride, const float* __restrict__ y,
                                                              long y_stride, const float* __restrict__ z, long z_stride,
                                                              const float* __restrict__ w, float eps, float mult, int size) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int base = blockIdx.y * size;
  const float* yr = y + t * y_stride + base;
  const float* zr = z + t * z_stride + base;
  float ss = 0.f;
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    const float v = yr[i] * silu_f(zr[i]);
    ss = fmaf(v, v, ss);
  }
  const float rinv = 1.0f / sqrtf(block_sum(ss, scratch) / size + eps);
  for (int i = threadIdx.x; i < size; i += blockDim.x) {
    const float v = yr[i] * silu_f(zr[i]);
    out[t * out_stride + base + i] = from_float<TO>(v * rinv * w[base + i] * mult);
  }
}

extern "C" int pi_gated_group_norm(void* out, int out_dtype, long out_stride, const float* y, long y_stride, const float* z,
                                   long z_stride, const float* w, float eps, float mult, int T, int width, int parts,
                                   hipStream_t stream) {
  PI_REQUIRE(T >= 0 && width > 0 && parts > 0 && parts <= 65535 && width % parts == 0, "gated norm: %d columns in %d parts", width, parts);
  if (T == 0) return 0;
  const int size = width / parts;
  const dim3 grid(T, parts), block(size >= 256 ? 256 : 64);
  if (out_dtype == PI_F32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, block, 0, stream, (float*)out, out_stride, y, y_stride, z, z_stride, w, eps, mult, size);
  else if (out_dtype == PI_BF16)
    hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, out_stride, y, y_stride, z, z_stride, w, eps, mult, size);
  else
    return pi_fail("gated norm: unsupported dtype %d", out_dtype);
  return pi_check_launch("gated_group_norm");
}

// ------------------------------------------------------------------ gated delta rule, a decay per key channel
// Per head h with key head g = h / (H / G), state S [d, dv] (float32, zero at the start):
//   q^ = q / sqrt(sum q^2 + unit_eps) * q_scale;  k^ = k / sqrt(sum k^2 + unit_eps);
//   decay[c] = exp(-exp(A_log[h]) * softplus(a[h, c] + dt_bias[h, c]));  beta = sigmoid(b[h]);
//   S <- diag(decay) S;  u = beta * (v - S^T k^);  S <- S + k^ u^T;  o = S^T q^
// q, k, v are columns of the convolution's output (q at 0, k at G * d, v at 2 * G * d).  A column
// of S never meets another column, so a wave walks its 16 columns alone; unit vectors, decays and
// beta of a chunk of tokens are made while the chunk is staged.
template <int NR>
__global__ __launch_bounds__(PI_WAVE) void delta_scan_kernel(
    float* __restrict__ o, long o_stride, const float* __restrict__ qkv, long qkv_stride, const float* __restrict__ a,
    long a_stride, const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ b, long b_stride,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ state, long state_stride, int H, int G,
    int d, int dv, float q_scale, float unit_eps) {
  constexpr int W = 4 * NR;
  __shared__ float sq[PI_SCAN_CHUNK][W], sk[PI_SCAN_CHUNK][W], sg[PI_SCAN_CHUNK][W], sv[PI_SCAN_CHUNK][PI_SCAN_COLUMNS], sbeta[PI_SCAN_CHUNK];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int col = blockIdx.z * PI_SCAN_COLUMNS + lane / 4, part = lane % 4;
  const int g = h / (H / G);
  const int qs = q_start[r], n = q_start[r + 1] - qs;
  if (n <= 0) return;
  float* S = state + (long)slots[r] * state_stride + (long)h * d * dv;
  const bool live = col < dv;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = part * NR + i;
    s[i] = (live && row < d) ? S[(long)row * dv + col] : 0.f;
  }
  const float A = expf(A_log[h]);
  const long q_col = (long)g * d, k_col = (long)G * d + (long)g * d, v_col = 2L * G * d + (long)h * dv + blockIdx.z * PI_SCAN_COLUMNS;
  for (int c0 = 0; c0 < n; c0 += PI_SCAN_CHUNK) {
    const int cn = n - c0 < PI_SCAN_CHUNK ? n - c0 : PI_SCAN_CHUNK;
    __syncthreads();
    for (int tt = 0; tt < cn; ++tt) {
      const long t = qs + c0 + tt;
      const float* src = qkv + t * qkv_stride;
      float q2 = 0.f, k2 = 0.f;
      for (int c = lane; c < d; c += PI_WAVE) {
        const float qv = src[q_col + c], kv = src[k_col + c];
        q2 = fmaf(qv, qv, q2);
        k2 = fmaf(kv, kv, k2);
      }
      const float qn = q_scale / sqrtf(wave_sum(q2) + unit_eps), kn = 1.0f / sqrtf(wave_sum(k2) + unit_eps);
      for (int c = lane; c < W; c += PI_WAVE) {
        const bool in = c < d;
        sq[tt][c] = in ? src[q_col + c] * qn : 0.f;
        sk[tt][c] = in ? src[k_col + c] * kn : 0.f;
        sg[tt][c] = in ? expf(-A * softplus_f(a[t * a_stride + (long)h * d + c] + dt_bias[(long)h * d + c])) : 0.f;
      }
      if (lane < PI_SCAN_COLUMNS) sv[tt][lane] = blockIdx.z * PI_SCAN_COLUMNS + lane < dv ? src[v_col + lane] : 0.f;
      if (lane == PI_SCAN_COLUMNS) sbeta[tt] = sigmoid_f(b[t * b_stride + h]);
    }
    __syncthreads();
    for (int tt = 0; tt < cn; ++tt) {
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        s[i] *= sg[tt][part * NR + i];
        dot = fmaf(s[i], sk[tt][part * NR + i], dot);
      }
      const float u = sbeta[tt] * (sv[tt][lane / 4] - quad_sum(dot));
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        s[i] = fmaf(sk[tt][part * NR + i], u, s[i]);
        acc = fmaf(s[i], sq[tt][part * NR + i], acc);
      }
      acc = quad_sum(acc);
      if (live && part == 0) o[(long)(qs + c0 + tt) * o_stride + (long)h * dv + col] = acc;
    }
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = part * NR + i;
    if (live && row < d) S[(long)row * dv + col] = s[i];
  }
}

extern "C" int pi_delta_scan(float* o, long o_stride, const float* qkv, long qkv_stride, const float* a, long a_stride,
                             const float* dt_bias, const float* A_log, const float* b, long b_stride, const int* q_start,
                             const int* slots, int R, float* state, long state_stride, int H, int G, int d, int dv, float q_scale,
                             float unit_eps, hipStream_t stream) {
  PI_REQUIRE(H > 0 && H <= 65535 && G > 0 && H % G == 0 && d > 0 && dv > 0, "delta rule: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d", H, G, d, dv);
  PI_REQUIRE(R >= 0 && state_stride >= (long)H * d * dv, "delta rule: a state row of %ld floats cannot hold %d x %d x %d", state_stride, H, d, dv);
  const int nr = scan_rows_per_lane(d);
  PI_REQUIRE(nr > 0, "delta rule: keys of %d channels are more than 256", d);
  if (R == 0) return 0;
  const dim3 grid(R, H, (dv + PI_SCAN_COLUMNS - 1) / PI_SCAN_COLUMNS), block(PI_WAVE);
#define PI_LAUNCH_DELTA(NR_)                                                                                                 \
  hipLaunchKernelGGL(delta_scan_kernel<NR_>, grid, block, 0, stream, o, o_stride, qkv, qkv_stride, a, a_stride, dt_bias,    \
                     A_log, b, b_stride, q_start, slots, state, state_stride, H, G, d, dv, q_scale, unit_eps)
  switch (nr) {
    case 4: PI_LAUNCH_DELTA(4); break;
    case 8: PI_LAUNCH_DELTA(8); break;
    case 16: PI_LAUNCH_DELTA(16); break;
    case 32: PI_LAUNCH_DELTA(32); break;
    default: PI_LAUNCH_DELTA(64); break;
  }
#undef PI_LAUNCH_DELTA
  return pi_check_launch("delta_scan");
}
