// A recurrent mixer with a matrix memory per head (the mLSTM cell of xLSTM), token by token.
//
// Per head, with state S [d, dv], n [d] and a running maximum m (all float32, zero at the
// start of a sequence), and per token the query q (already scaled), key k, value v and the two
// gate pre-activations zi, zf (biases added here):
//   i = cap * tanh(zi / cap)                     log input gate
//   f = logsigmoid(cap * tanh(zf / cap))         log forget gate
//   m' = max(f + m, i);  a = exp(f + m - m');  b = exp(i - m')
//   S' = a S + b k v^T;  n' = a n + b k
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// The scan is sequential in the tokens of a request and runs them in the order given, so its
// result for a token does not depend on how the tokens were cut into steps.
//
// One wave per (request, head, 16 value columns): lane = column + 16 * part; the four parts split
// the d rows of the state, which stays in registers over all tokens of the step.  n and m are kept
// once per group of 16 columns ([slices, d + 1] per head), so that no block reads what another writes.
//
// State row of one request (floats): [heads][d][dv] S, then [heads][slices][d + 1] (n, then m).
#include "common.h"

#define MM_COLS 16
#define MM_PARTS 4

__host__ __device__ inline long mm_state_floats(int heads, int d, int dv) {
  const int slices = (dv + MM_COLS - 1) / MM_COLS;
  return (long)heads * d * dv + (long)heads * slices * (d + 1);
}

extern "C" long pi_matrix_memory_state_floats(int heads, int d, int dv) { return mm_state_floats(heads, d, dv); }

template <int DPP>
__global__ __launch_bounds__(PI_WAVE) void matrix_memory_scan_kernel(
    float* __restrict__ out, long out_stride, const float* __restrict__ proj, long proj_stride, int q_off, int k_off, int v_off,
    int i_off, int f_off, const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale,
    const int* __restrict__ q_start, const int* __restrict__ slots, float* __restrict__ state, long state_stride, int max_slots,
    int heads, int d, int dv) {
  const int r = blockIdx.x, h = blockIdx.y, slice = blockIdx.z;
  const int lane = threadIdx.x, col = lane % MM_COLS, part = lane / MM_COLS;
  const int c = slice * MM_COLS + col;
  const bool col_ok = c < dv;
  const int slot = slots[r];
  if (slot < 0 || slot >= max_slots) return;
  const int slices = gridDim.z;
  float* Sg = state + (long)slot * state_stride + (long)h * d * dv;
  float* nm = state + (long)slot * state_stride + (long)heads * d * dv + ((long)h * slices + slice) * (d + 1);
  const int r0 = part * DPP;                     // this lane's rows of the state: r0 .. r0 + DPP - 1 (those below d)
  float S[DPP], n[DPP];
#pragma unroll
  for (int i = 0; i < DPP; ++i) {
    const bool ok = r0 + i < d;
    S[i] = (ok && col_ok) ? Sg[(long)(r0 + i) * dv + c] : 0.f;
    n[i] = ok ? nm[r0 + i] : 0.f;
  }
  float m = nm[d];
  const int t0 = q_start[r], t1 = q_start[r + 1];
  for (int t = t0; t < t1; ++t) {
    const float* row = proj + (long)t * proj_stride;
    const float zi = row[i_off + h] + i_bias[h], zf = row[f_off + h] + f_bias[h];
    const float ig = cap * tanhf(zi / cap);
    const float fz = cap * tanhf(zf / cap);
    const float fg = fminf(fz, 0.f) - log1pf(expf(-fabsf(fz)));
    const float m_new = fmaxf(fg + m, ig);
    const float a = expf(fg + m - m_new), b = expf(ig - m_new);
    const float v = col_ok ? row[v_off + h * dv + c] : 0.f;
    const float bv = b * v;
    const float* qr = row + q_off + h * d + r0;
    const float* kr = row + k_off + h * d + r0;
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int i = 0; i < DPP; ++i) {
      if (r0 + i < d) {
        const float kk = kr[i], qq = qr[i] * q_scale;
        S[i] = fmaf(a, S[i], kk * bv);
        n[i] = fmaf(a, n[i], b * kk);
        num = fmaf(S[i], qq, num);
        den = fmaf(n[i], qq, den);
      }
    }
    num += __shfl_xor(num, 16, PI_WAVE);
    den += __shfl_xor(den, 16, PI_WAVE);
    num += __shfl_xor(num, 32, PI_WAVE);
    den += __shfl_xor(den, 32, PI_WAVE);
    m = m_new;
    if (part == 0 && col_ok) out[(long)t * out_stride + h * dv + c] = num / (fmaxf(fabsf(den), expf(-m_new)) + 1e-6f);
  }
#pragma unroll
  for (int i = 0; i < DPP; ++i) {
    if (r0 + i < d) {
      if (col_ok) Sg[(long)(r0 + i) * dv + c] = S[i];
      if (col == 0) nm[r0 + i] = n[i];
    }
  }
  if (lane == 0) nm[d] = m;
}

// out float32 [T, heads * dv]: the cell's raw output per head.  proj float32 rows hold q, k
// ([heads, d] each), v ([heads, dv]) and the gate pre-activations ([heads] each) at the given
// column offsets.  Requests r = 0 .. R-1 own tokens q_start[r] .. q_start[r+1]; their states are
// rows slots[r] of `state`.
extern "C" int pi_matrix_memory_scan(float* out, long out_stride, const float* proj, long proj_stride, int q_off, int k_off,
                                     int v_off, int i_off, int f_off, const float* i_bias, const float* f_bias, float cap,
                                     float q_scale, const int* q_start, const int* slots, int R, float* state,
                                     long state_stride, int max_slots, int heads, int d, int dv, hipStream_t stream) {
  PI_REQUIRE(R >= 0 && heads > 0 && d > 0 && dv > 0, "matrix memory: bad sizes");
  PI_REQUIRE(d <= 4 * 64, "matrix memory: key size %d is above %d", d, 4 * 64);
  PI_REQUIRE(state_stride >= mm_state_floats(heads, d, dv), "matrix memory: state rows of %ld floats are too short", state_stride);
  PI_REQUIRE(cap > 0.f, "matrix memory: the gates' cap must be positive");
  PI_REQUIRE(heads <= 65535, "matrix memory: too many heads");
  if (R == 0) return 0;
  const int slices = (dv + MM_COLS - 1) / MM_COLS;
  PI_REQUIRE(slices <= 65535, "matrix memory: value size %d is too large", dv);
  const dim3 grid(R, heads, slices), block(PI_WAVE);
  const int dpp = (d + MM_PARTS - 1) / MM_PARTS;
#define MM_GO(DPP) hipLaunchKernelGGL(matrix_memory_scan_kernel<DPP>, grid, block, 0, stream, out, out_stride, proj, proj_stride, q_off, \
                                      k_off, v_off, i_off, f_off, i_bias, f_bias, cap, q_scale, q_start, slots, state, state_stride,    \
                                      max_slots, heads, d, dv)
  if (dpp <= 8) MM_GO(8);
  else if (dpp <= 16) MM_GO(16);
  else if (dpp <= 32) MM_GO(32);
  else MM_GO(64);
#undef MM_GO
  return pi_check_launch("matrix_memory_scan");
}

// y[t, h*dv + c] = o / sqrt(mean_c(o^2) + eps) * w[h*dv + c] * sigmoid(g[t, h*dv + c]); one wave per (token, head)
template <typename T>
__global__ __launch_bounds__(PI_WAVE) void head_norm_gate_kernel(T* __restrict__ y, const float* __restrict__ o, long o_stride,
                                                                 const float* __restrict__ g, long g_stride,
                                                                 const float* __restrict__ w, float eps, int heads, int dv) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + t * o_stride + (long)h * dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += PI_WAVE) ss = fmaf(orow[c], orow[c], ss);
  const float r = 1.0f / sqrtf(wave_sum(ss) / dv + eps);
  for (int c = lane; c < dv; c += PI_WAVE) {
    const float gate = 1.0f / (1.0f + expf(-g[t * g_stride + h * dv + c]));
    y[(t * heads + h) * dv + c] = from_float<T>(orow[c] * r * w[h * dv + c] * gate);
  }
}

extern "C" int pi_head_norm_gate(void* y, int dtype, const float* o, long o_stride, const float* g, long g_stride,
                                 const float* w, float eps, int T, int heads, int dv, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && heads > 0 && heads <= 65535 && dv > 0, "head norm: bad sizes");
  if (T == 0) return 0;
  const dim3 grid(T, heads), block(PI_WAVE);
  if (dtype == PI_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, stream, (float*)y, o, o_stride, g, g_stride, w, eps, heads, dv);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, o, o_stride, g, g_stride, w, eps, heads, dv);
  else
    return pi_fail("head norm: unsupported dtype %d", dtype);
  return pi_check_launch("head_norm_gate");
}
