// The gated delta rule with one decay per head and key channel, and what surrounds it: the short causal convolution
// over time with its carried inputs, the unit vectors, decays and write strengths, the recurrence over a request's
// tokens with the state carried in its slot, and the gated RMS norm of the read-out.
//
// Per head, with S [D key channels][E value channels] (float, one per request and head):
//   S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
// Column j of S only ever meets column j of v and o, so the columns of a head are independent chains: a thread owns 16
// key channels of one column in registers, the RG = D/16 threads of a column sit in neighbouring lanes and add their
// parts of the two dot products by lane exchange, and nothing waits at a barrier.  Everything here is 32-bit.
//
// A request's slot holds S [H][D][E] and behind it the last K - 1 inputs of the convolution [K - 1][C] (oldest first).
#include "common.h"

#define ND_MAX_TAPS 16
#define ND_ROWS 16  // key channels of a column that one thread owns

// ------------------------------------------------------------------------------------------------
// y[r][c] = silu(sum_j taps[c][j] * in(i - (K-1) + j)),  i the token's index among its request's tokens of this step;
// in(t) is this step's input for t >= 0 and the carried input K-1+t for t < 0.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void conv_silu_kernel(float* __restrict__ out, const T* __restrict__ x, int x_stride, const float* __restrict__ taps,
                                 const float* __restrict__ state, size_t slot_stride, size_t conv_off, const int* __restrict__ token_req,
                                 const int* __restrict__ qo_indptr, const int* __restrict__ state_slots, int C, int K) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = token_req[r];
  const int i = r - qo_indptr[b];
  const float* carried = state + (size_t)state_slots[b] * slot_stride + conv_off;
  float y = 0.f;
  for (int j = 0; j < K; ++j) {
    const int t = i - (K - 1) + j;
    const float v = t >= 0 ? to_f(x[(size_t)(r - (K - 1) + j) * x_stride + c]) : carried[(size_t)(K - 1 + t) * C + c];
    y = fmaf(taps[(size_t)c * K + j], v, y);
  }
  out[(size_t)r * C + c] = y / (1.f + expf(-y));
}

// After the convolution has read them: the carried inputs become the last K-1 inputs including this step's.
template <typename T>
__global__ void conv_carry_kernel(const T* __restrict__ x, int x_stride, float* __restrict__ state, size_t slot_stride, size_t conv_off,
                                  const int* __restrict__ qo_indptr, const int* __restrict__ state_slots, int C, int K) {
  const int b = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r0 = qo_indptr[b], L = qo_indptr[b + 1] - r0;
  if (L <= 0) return;
  float* carried = state + (size_t)state_slots[b] * slot_stride + conv_off;
  float old[ND_MAX_TAPS];
  for (int j = 0; j < K - 1; ++j) old[j] = carried[(size_t)j * C + c];
  for (int j = 0; j < K - 1; ++j) {
    const int t = L - (K - 1) + j;
    carried[(size_t)j * C + c] = t >= 0 ? to_f(x[(size_t)(r0 + t) * x_stride + c]) : old[K - 1 + t];
  }
}

extern "C" int ns_conv_silu_carry(float* out, const void* x, int x_stride, const float* taps, float* state, size_t slot_stride,
                                  size_t conv_off, const int* token_req, const int* qo_indptr, const int* state_slots, int n_tokens,
                                  int n_reqs, int C, int K, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || n_reqs <= 0 || n_reqs > 65535 || C <= 0 || K < 1 || K > ND_MAX_TAPS) return NS_ERR_BAD_ARG;
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
  const int bx = (C + 255) / 256;
  if (bx > 65535) return NS_ERR_BAD_ARG;
  {
    dim3 grid(n_tokens, bx);
    if (dtype == NS_DTYPE_F32)
      conv_silu_kernel<float><<<grid, 256, 0, stream>>>(out, (const float*)x, x_stride, taps, state, slot_stride, conv_off, token_req,
                                                         qo_indptr, state_slots, C, K);
    else
      conv_silu_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, (const bf16_t*)x, x_stride, taps, state, slot_stride, conv_off, token_req,
                                                          qo_indptr, state_slots, C, K);
  }
  if (K > 1) {
    dim3 grid(bx, n_reqs);
    if (dtype == NS_DTYPE_F32)
      conv_carry_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, state, slot_stride, conv_off, qo_indptr, state_slots, C, K);
    else
      conv_carry_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, state, slot_stride, conv_off, qo_indptr, state_slots, C, K);
  }
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Per token: q and k of every key/value head become unit vectors, x / sqrt(sum(x^2) + 1e-6), q times D^(-1/2), in
// place in qkv [n][2 G D + H E]; g = exp(-exp(A_log[h]) softplus(a + dt_bias)) [n][H D]; beta = sigmoid(b) [n][H].
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T>
__global__ void delta_prep_kernel(float* __restrict__ qkv, int C, float* __restrict__ g, float* __restrict__ beta, const T* __restrict__ a,
                                  int a_stride, const T* __restrict__ bp, int b_stride, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, int H, int G, int D) {
  const int r = blockIdx.x, lane = threadIdx.x & (NS_WAVE - 1), wave = threadIdx.x / NS_WAVE, nw = blockDim.x / NS_WAVE;
  float* row = qkv + (size_t)r * C;
  const float q_scale = 1.f / sqrtf((float)D);
  for (int vec = wave; vec < 2 * G; vec += nw) {  // q heads, then k heads
    float* p = row + (size_t)vec * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += NS_WAVE) ss = fmaf(p[d], p[d], ss);
    ss = wave_sum(ss);
    const float f = (vec < G ? q_scale : 1.f) / sqrtf(ss + 1e-6f);
    for (int d = lane; d < D; d += NS_WAVE) p[d] *= f;
  }
  for (int i = threadIdx.x; i < H * D; i += blockDim.x) {
    const float z = to_f(a[(size_t)r * a_stride + i]) + dt_bias[i];
    g[(size_t)r * H * D + i] = expf(-expf(a_log[i / D]) * softplus_f(z));
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) beta[(size_t)r * H + h] = 1.f / (1.f + expf(-to_f(bp[(size_t)r * b_stride + h])));
}

extern "C" int ns_delta_prep(float* qkv, int C, float* g, float* beta, const void* a, int a_stride, const void* bp, int b_stride,
                             const float* dt_bias, const float* a_log, int n_tokens, int H, int G, int D, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || C < 2 * G * D) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    delta_prep_kernel<float><<<n_tokens, 256, 0, stream>>>(qkv, C, g, beta, (const float*)a, a_stride, (const float*)bp, b_stride, dt_bias,
                                                            a_log, H, G, D);
  else if (dtype == NS_DTYPE_BF16)
    delta_prep_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(qkv, C, g, beta, (const bf16_t*)a, a_stride, (const bf16_t*)bp, b_stride,
                                                             dt_bias, a_log, H, G, D);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// The recurrence.  grid (requests, heads, blocks of columns); a thread = (column jl of the block, row group rg), lane
// = jl * RG + rg, RG a power of two (at most 64) with 16 RG >= D.  Channels beyond D carry zeros.
// ------------------------------------------------------------------------------------------------
struct DeltaVec {
  float v[ND_ROWS];
};

__device__ __forceinline__ void delta_load(DeltaVec& out, const float* p, int valid, bool vec4) {
  if (vec4 && valid == ND_ROWS) {
    const float4* p4 = reinterpret_cast<const float4*>(p);
#pragma unroll
    for (int i = 0; i < ND_ROWS / 4; ++i) {
      const float4 t = p4[i];
      out.v[4 * i] = t.x, out.v[4 * i + 1] = t.y, out.v[4 * i + 2] = t.z, out.v[4 * i + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < ND_ROWS; ++i) out.v[i] = i < valid ? p[i] : 0.f;
  }
}

__device__ __forceinline__ float group_sum(float v, int rg_count) {
  for (int o = 1; o < rg_count; o <<= 1) v += __shfl_xor(v, o, NS_WAVE);
  return v;
}

__global__ __launch_bounds__(256) void delta_scan_kernel(float* __restrict__ o, const float* __restrict__ qkv, int C,
                                                         const float* __restrict__ g, const float* __restrict__ beta,
                                                         float* __restrict__ state, size_t slot_stride, const int* __restrict__ qo_indptr,
                                                         const int* __restrict__ state_slots, int H, int G, int D, int E, int RG, int vec4) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int r0 = qo_indptr[b], r1 = qo_indptr[b + 1];
  if (r1 <= r0) return;
  const int cols = blockDim.x / RG;
  const int jl = threadIdx.x / RG, rg = threadIdx.x % RG;
  const int j = blockIdx.z * cols + jl;
  const bool col_ok = j < E;
  const int d0 = rg * ND_ROWS;
  const int valid = max(0, min(ND_ROWS, D - d0));
  const int kh = h / (H / G);
  float* S = state + (size_t)state_slots[b] * slot_stride + (size_t)h * D * E;
  float s[ND_ROWS];
#pragma unroll
  for (int i = 0; i < ND_ROWS; ++i) s[i] = (col_ok && i < valid) ? S[(size_t)(d0 + i) * E + j] : 0.f;
  const size_t q_off = (size_t)kh * D + d0, k_off = (size_t)G * D + (size_t)kh * D + d0, v_off = (size_t)2 * G * D + (size_t)h * E + (col_ok ? j : 0);
  const size_t g_off = (size_t)h * D + d0;
  const bool v4 = vec4 != 0;
  DeltaVec qn, kn, gn;
  float vn, bn;
  {
    const float* row = qkv + (size_t)r0 * C;
    delta_load(qn, row + q_off, valid, v4);
    delta_load(kn, row + k_off, valid, v4);
    delta_load(gn, g + (size_t)r0 * H * D + g_off, valid, v4);
    vn = row[v_off];
    bn = beta[(size_t)r0 * H + h];
  }
  for (int r = r0; r < r1; ++r) {
    const DeltaVec qc = qn, kc = kn, gc = gn;
    const float vc = vn, bc = bn;
    if (r + 1 < r1) {  // the next token's operands are on their way while this one's chain runs
      const float* row = qkv + (size_t)(r + 1) * C;
      delta_load(qn, row + q_off, valid, v4);
      delta_load(kn, row + k_off, valid, v4);
      delta_load(gn, g + (size_t)(r + 1) * H * D + g_off, valid, v4);
      vn = row[v_off];
      bn = beta[(size_t)(r + 1) * H + h];
    }
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < ND_ROWS; ++i) {
      s[i] *= gc.v[i];
      dot = fmaf(kc.v[i], s[i], dot);
    }
    dot = group_sum(dot, RG);
    const float u = bc * (vc - dot);
    float out = 0.f;
#pragma unroll
    for (int i = 0; i < ND_ROWS; ++i) {
      s[i] = fmaf(kc.v[i], u, s[i]);
      out = fmaf(qc.v[i], s[i], out);
    }
    out = group_sum(out, RG);
    if (rg == 0 && col_ok) o[(size_t)r * H * E + (size_t)h * E + j] = out;
  }
#pragma unroll
  for (int i = 0; i < ND_ROWS; ++i)
    if (col_ok && i < valid) S[(size_t)(d0 + i) * E + j] = s[i];
}

extern "C" int ns_delta_scan(float* o, const float* qkv, int C, const float* g, const float* beta, float* state, size_t slot_stride,
                             const int* qo_indptr, const int* state_slots, int n_reqs, int H, int G, int D, int E, hipStream_t stream) {
  if (n_reqs <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > ND_ROWS * NS_WAVE || E <= 0 || H > 65535) return NS_ERR_BAD_ARG;
  int RG = 1;
  while (RG * ND_ROWS < D) RG *= 2;
  const int cols = 256 / RG;
  const int zb = (E + cols - 1) / cols;
  if (zb > 65535) return NS_ERR_BAD_ARG;
  // 16-byte loads where every vector a thread reads starts at a multiple of four floats
  const int vec4 = (D % 4 == 0 && C % 4 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)g % 16) == 0) ? 1 : 0;
  delta_scan_kernel<<<dim3(n_reqs, H, zb), 256, 0, stream>>>(o, qkv, C, g, beta, state, slot_stride, qo_indptr, state_slots, H, G, D, E, RG,
                                                              vec4);
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// out[r][h][:] = o / sqrt(mean(o^2) + eps) * w[:] * sigmoid(gate[r][h][:]),  o float, gate and out in the model's type.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void gated_rms_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate, int gate_stride,
                                 const float* __restrict__ w, int H, int E, float eps) {
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* p = o + ((size_t)r * H + h) * E;
  float ss = 0.f;
  for (int e = lane; e < E; e += NS_WAVE) ss = fmaf(p[e], p[e], ss);
  ss = wave_sum(ss);
  const float rinv = 1.f / sqrtf(ss / (float)E + eps);
  for (int e = lane; e < E; e += NS_WAVE) {
    const float z = to_f(gate[(size_t)r * gate_stride + (size_t)h * E + e]);
    out[((size_t)r * H + h) * E + e] = from_f<T>(p[e] * rinv * w[e] / (1.f + expf(-z)));
  }
}

extern "C" int ns_gated_rms(void* out, const float* o, const void* gate, int gate_stride, const float* w, int n_tokens, int H, int E,
                            float eps, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || H <= 0 || H > 65535 || E <= 0) return NS_ERR_BAD_ARG;
  dim3 grid(n_tokens, H);
  if (dtype == NS_DTYPE_F32)
    gated_rms_kernel<float><<<grid, NS_WAVE, 0, stream>>>((float*)out, o, (const float*)gate, gate_stride, w, H, E, eps);
  else if (dtype == NS_DTYPE_BF16)
    gated_rms_kernel<bf16_t><<<grid, NS_WAVE, 0, stream>>>((bf16_t*)out, o, (const bf16_t*)gate, gate_stride, w, H, E, eps);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
