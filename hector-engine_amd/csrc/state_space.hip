// Kernels of a state-space mixer (a selective scan with a short causal convolution in front and a
// gated, grouped RMS norm behind), over the packed rows of a step. What a sequence carries from step
// to step lives in its row of the cache's state area, in fp32: the last K-1 inputs of the
// convolution, [K-1][C], and then the state of the scan, [R][P][Npad] (head, value dim, state dim
// padded to the threads' share). Everything that enters the recurrence is fp32.
#include "common.h"
#include "hector_kernels.h"

__device__ __forceinline__ float ss_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float ss_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---- causal convolution per channel ---------------------------------------------------------
// out[row, c] = silu(bias[c] + sum_j taps[c, j] * u[pos - (K-1) + j, c]): the last tap weighs the
// row's own input. Inputs before the step's first row of the sequence come from the carried inputs
// (zeros at a sequence's start). SINGLE: every sequence brings one row, and the thread that computed
// (row, c) also moves the carried inputs on; otherwise conv_carry_kernel does that afterwards.
template <typename T, bool SINGLE>
__global__ void conv_taps_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t x_stride,
                                 const void* __restrict__ taps, const void* __restrict__ bias, int w_dtype,
                                 uint8_t* __restrict__ state, int64_t state_stride,
                                 const int32_t* __restrict__ positions, const int32_t* __restrict__ row_seq,
                                 const int32_t* __restrict__ seq_slot, const int32_t* __restrict__ seq_start,
                                 int C, int K) {
  const int64_t row = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int seq = row_seq[row];
  const int slot = seq < 0 ? -1 : seq_slot[seq];
  if (slot < 0) {   // a padding row stays finite
    out[row * (int64_t)C + c] = from_float<T>(0.f);
    return;
  }
  const int before = positions[row] - seq_start[seq];   // rows of the same sequence ahead of this one in the step
  float* hist = reinterpret_cast<float*>(state + (int64_t)slot * state_stride);
  float acc = load_param(bias, c, w_dtype);
  for (int j = 0; j < K; ++j) {
    const int back = K - 1 - j;
    float u;
    if (back <= before)
      u = to_float(x[(row - back) * x_stride + c]);
    else
      u = hist[(int64_t)(K - 1 - (back - before)) * C + c];
    acc = fmaf(load_param(taps, (int64_t)c * K + j, w_dtype), u, acc);
  }
  out[row * (int64_t)C + c] = from_float<T>(ss_silu(acc));
  if (SINGLE) {
    for (int i = 0; i + 2 < K; ++i) hist[(int64_t)i * C + c] = hist[(int64_t)(i + 1) * C + c];
    if (K > 1) hist[(int64_t)(K - 2) * C + c] = to_float(x[row * x_stride + c]);
  }
}

// The carried inputs after a step: the last K-1 inputs of the sequence, from its new rows and, where
// those are fewer, from what was carried before. One thread owns (sequence, channel).
template <typename T>
__global__ void conv_carry_kernel(const T* __restrict__ x, int64_t x_stride, uint8_t* __restrict__ state,
                                  int64_t state_stride, const int32_t* __restrict__ cu_seqlens,
                                  const int32_t* __restrict__ seq_slot, int C, int K) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int end = cu_seqlens[seq + 1];
  const int n = end - cu_seqlens[seq];
  if (n <= 0) return;
  float* hist = reinterpret_cast<float*>(state + (int64_t)slot * state_stride);
  // entry i comes from entry i + n or from a new row: entries are read before they are written
  for (int i = 0; i < K - 1; ++i) {
    const int back = K - 1 - i;
    hist[(int64_t)i * C + c] = back <= n ? to_float(x[(int64_t)(end - back) * x_stride + c])
                                         : hist[(int64_t)(i + n) * C + c];
  }
}

extern "C" int he_conv_state(void* out, const void* x, int64_t x_stride, const void* taps, const void* bias,
                             int w_dtype, void* state, int64_t state_stride, const void* positions,
                             const void* row_seq, const void* seq_slot, const void* seq_start,
                             const void* cu_seqlens, int rows, int num_seqs, int C, int K, int all_single,
                             int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && num_seqs >= 0 && C > 0 && K >= 1 && K <= 64, "he_conv_state: bad sizes rows=%d C=%d K=%d", rows,
             C, K);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_conv_state: unknown dtype %d", dtype);
  HE_REQUIRE(state != nullptr && state_stride >= (int64_t)(K - 1) * C * 4 && state_stride % 4 == 0,
             "he_conv_state: the state row is too short for %d x %d carried inputs", K - 1, C);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = C >= 256 ? 256 : 64;
  const dim3 grid((C + threads - 1) / threads, rows);
#define CONV_LAUNCH(T, SINGLE)                                                                          \
  conv_taps_kernel<T, SINGLE><<<grid, threads, 0, s>>>(                                                 \
      (T*)out, (const T*)x, x_stride, taps, bias, w_dtype, (uint8_t*)state, state_stride,               \
      (const int32_t*)positions, (const int32_t*)row_seq, (const int32_t*)seq_slot, (const int32_t*)seq_start, C, K)
  if (dtype == HE_BF16) {
    if (all_single) CONV_LAUNCH(bf16_t, true); else CONV_LAUNCH(bf16_t, false);
  } else {
    if (all_single) CONV_LAUNCH(float, true); else CONV_LAUNCH(float, false);
  }
#undef CONV_LAUNCH
  int st = he_check_launch("he_conv_state");
  if (st || all_single || num_seqs == 0 || K == 1) return st;
  const dim3 cgrid((C + threads - 1) / threads, num_seqs);
  if (dtype == HE_BF16)
    conv_carry_kernel<bf16_t><<<cgrid, threads, 0, s>>>((const bf16_t*)x, x_stride, (uint8_t*)state, state_stride,
                                                        (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, C, K);
  else
    conv_carry_kernel<float><<<cgrid, threads, 0, s>>>((const float*)x, x_stride, (uint8_t*)state, state_stride,
                                                       (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, C, K);
  return he_check_launch("he_conv_state (carry)");
}

// ---- selective scan ---------------------------------------------------------------------------
// Per head r (its B and C vectors are those of group r / (R / Q)) and token t:
//   dt = softplus(dt_in + dt_bias_r),  S <- exp(-exp(A_log_r) dt) S + dt B x^T,  y = S^T C + D_r x
// with S [N][P] carried in fp32. A thread holds NPT neighbouring state dims of one value dim p; the NG
// threads of a p are neighbouring lanes, and their partial sums of y meet in a butterfly whose order
// does not depend on the step. A workgroup takes PB value dims of one (sequence, head) and walks the
// sequence's rows in order.
static inline int ss_npt(int N) { return N <= 64 ? 8 : 16; }
static inline int ss_groups(int N) {
  const int npt = ss_npt(N);
  int ng = 1;
  while (ng * npt < N) ng *= 2;
  return ng;
}

template <typename T, int NPT>
__global__ __launch_bounds__(256) void ssm_scan_kernel(
    float* __restrict__ y, const T* __restrict__ xbc, const T* __restrict__ dt_in, int64_t dt_stride,
    const void* __restrict__ dt_bias, const void* __restrict__ a_log, const void* __restrict__ d_skip, int w_dtype,
    uint8_t* __restrict__ state, int64_t state_stride, int64_t state_offset, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ seq_slot, int R, int Q, int N, int P, int NG, int PB) {
  const int seq = blockIdx.z, r = blockIdx.y;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
  if (t1 <= t0) return;
  const int ng = threadIdx.x % NG;
  const int p_raw = blockIdx.x * PB + threadIdx.x / NG;
  const bool live = p_raw < P;
  const int p = live ? p_raw : P - 1;
  const int n0 = ng * NPT;
  const int Npad = NG * NPT;
  const int inner = R * P;
  const int C = inner + 2 * Q * N;
  const int q = r / (R / Q);
  float* S = reinterpret_cast<float*>(state + (int64_t)slot * state_stride + state_offset) +
             ((int64_t)r * P + p) * Npad + n0;
  float s[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) s[i] = S[i];
  const float a = -expf(load_param(a_log, r, w_dtype));
  const float dk = load_param(d_skip, r, w_dtype);
  const float db = load_param(dt_bias, r, w_dtype);
  for (int t = t0; t < t1; ++t) {
    const T* row = xbc + (int64_t)t * C;
    const float x = to_float(row[r * P + p]);
    const float dt = ss_softplus(to_float(dt_in[(int64_t)t * dt_stride + r]) + db);
    const float decay = expf(a * dt);
    const float dtx = dt * x;
    const T* Bv = row + inner + q * N;
    const T* Cv = Bv + Q * N;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NPT; ++i) {
      const int n = n0 + i;
      const float b = n < N ? to_float(Bv[n]) : 0.f;
      const float c = n < N ? to_float(Cv[n]) : 0.f;
      s[i] = fmaf(decay, s[i], dtx * b);
      acc = fmaf(s[i], c, acc);
    }
    for (int m = 1; m < NG; m <<= 1) acc += __shfl_xor(acc, m);
    if (ng == 0 && live) y[(int64_t)t * inner + r * P + p] = fmaf(dk, x, acc);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NPT; ++i) S[i] = s[i];
  }
}

extern "C" int64_t he_ssm_state_floats(int R, int P, int N) {
  if (R <= 0 || P <= 0 || N <= 0) return 0;
  return (int64_t)R * P * ss_groups(N) * ss_npt(N);
}

extern "C" int he_ssm_scan(void* y_f32, const void* xbc, const void* dt_in, int64_t dt_stride, const void* dt_bias,
                           const void* a_log, const void* d_skip, int w_dtype, void* state, int64_t state_stride,
                           int64_t state_offset, const void* cu_seqlens, const void* seq_slot, int rows, int num_seqs,
                           int R, int Q, int N, int P, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && num_seqs >= 0 && R > 0 && Q > 0 && N > 0 && P > 0 && R % Q == 0,
             "he_ssm_scan: bad sizes R=%d Q=%d N=%d P=%d", R, Q, N, P);
  HE_REQUIRE(N <= 1024, "he_ssm_scan: state size %d above 1024", N);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_ssm_scan: unknown dtype %d", dtype);
  HE_REQUIRE(state != nullptr && state_offset % 16 == 0 && state_stride % 16 == 0 &&
                 state_stride >= state_offset + 4 * he_ssm_state_floats(R, P, N),
             "he_ssm_scan: the state row is too short or not aligned");
  if (rows == 0 || num_seqs == 0) return 0;
  const int NG = ss_groups(N);
  const int PB = 256 / NG < P ? 256 / NG : P;
  const int threads = (PB * NG + 63) / 64 * 64;
  const dim3 grid((P + PB - 1) / PB, R, num_seqs);
  hipStream_t s = (hipStream_t)stream;
#define SCAN_LAUNCH(T, NPT)                                                                                   \
  ssm_scan_kernel<T, NPT><<<grid, threads, 0, s>>>(                                                           \
      (float*)y_f32, (const T*)xbc, (const T*)dt_in, dt_stride, dt_bias, a_log, d_skip, w_dtype, (uint8_t*)state, \
      state_stride, state_offset, (const int32_t*)cu_seqlens, (const int32_t*)seq_slot, R, Q, N, P, NG, PB)
  if (dtype == HE_BF16) {
    if (ss_npt(N) == 8) SCAN_LAUNCH(bf16_t, 8); else SCAN_LAUNCH(bf16_t, 16);
  } else {
    if (ss_npt(N) == 8) SCAN_LAUNCH(float, 8); else SCAN_LAUNCH(float, 16);
  }
#undef SCAN_LAUNCH
  return he_check_launch("he_ssm_scan");
}

// ---- gated, grouped RMS norm ------------------------------------------------------------------
// out[row, c] = v / sqrt(mean over c's part of v^2 + eps) * weight[c], v = y[row, c] * silu(z[row, c]):
// the gate comes before the norm, and each of the `parts` equal stretches of a row has a root mean
// square of its own. One workgroup a (row, part).
template <typename T>
__global__ void gated_group_norm_kernel(T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ z,
                                        int64_t z_stride, const void* __restrict__ weight, int w_dtype, int W,
                                        int parts, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.y;
  const int width = W / parts;
  const int c0 = blockIdx.x * width;
  float sq = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = y[row * W + c0 + i] * ss_silu(to_float(z[row * z_stride + c0 + i]));
    sq = fmaf(v, v, sq);
  }
  const float total = block_sum(sq, scratch);
  const float inv = 1.f / sqrtf(total / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = y[row * W + c0 + i] * ss_silu(to_float(z[row * z_stride + c0 + i]));
    out[row * W + c0 + i] = from_float<T>(v * inv * load_param(weight, c0 + i, w_dtype));
  }
}

extern "C" int he_gated_group_norm(void* out, const void* y_f32, const void* z, int64_t z_stride, const void* weight,
                                   int w_dtype, int rows, int W, int parts, float eps, int dtype, void* stream) {
  HE_REQUIRE(rows >= 0 && W > 0 && parts > 0 && W % parts == 0, "he_gated_group_norm: bad sizes W=%d parts=%d", W, parts);
  HE_REQUIRE(dtype == HE_BF16 || dtype == HE_F32, "he_gated_group_norm: unknown dtype %d", dtype);
  if (rows == 0) return 0;
  const int width = W / parts;
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  const dim3 grid(parts, rows);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HE_BF16)
    gated_group_norm_kernel<bf16_t><<<grid, threads, 0, s>>>((bf16_t*)out, (const float*)y_f32, (const bf16_t*)z, z_stride,
                                                             weight, w_dtype, W, parts, eps);
  else
    gated_group_norm_kernel<float><<<grid, threads, 0, s>>>((float*)out, (const float*)y_f32, (const float*)z, z_stride,
                                                            weight, w_dtype, W, parts, eps);
  return he_check_launch("he_gated_group_norm");
}
