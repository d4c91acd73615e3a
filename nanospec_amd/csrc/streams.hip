// A residual stream that is kept in 32-bit whatever the model computes in, and that may be several parallel streams
// (hyper-connections): x [tokens][S][W], float.  A sublayer reads one mix of the streams through an RMS norm and
// writes its output back into all of them while the streams are mixed among themselves:
//   read:   u = sum_s a[s] x_s;            h = w * u / sqrt(mean(u^2) + eps)      (h in the model's precision)
//   write:  x_t <- sum_s M[s][t] x_s + c[t] y     for all t at once, from the old streams
// S = 1 with a = M = 1 is the plain pre-norm residual x <- x + c y with its sum in 32-bit.
#include "common.h"

#define NS_MAX_STREAMS 16

// out[i][s][:] = table[ids[i]][:] * scale for every copy s
template <typename T>
__global__ void embed_streams_kernel(float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids, int hidden,
                                     int copies, float scale) {
  const int row = blockIdx.x;
  const T* src = table + (size_t)ids[row] * hidden;
  float* dst = out + (size_t)row * copies * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = to_f(src[i]) * scale;
    for (int s = 0; s < copies; ++s) dst[(size_t)s * hidden + i] = v;
  }
}

extern "C" int ns_embed_streams(float* out, const void* table, const int* ids, int n_tokens, int hidden, int copies, float scale,
                                int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || hidden <= 0 || copies <= 0 || copies > NS_MAX_STREAMS) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    embed_streams_kernel<float><<<n_tokens, 256, 0, stream>>>(out, (const float*)table, ids, hidden, copies, scale);
  else if (dtype == NS_DTYPE_BF16)
    embed_streams_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(out, (const bf16_t*)table, ids, hidden, copies, scale);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// One workgroup a row.  The mix u is formed twice (once for the sum of squares, once for the output) in the same order,
// so a row costs two reads of S*W floats from cache and no scratch.  ``sum_out`` (optional): the mix itself, float.
template <typename T>
__global__ void stream_read_norm_kernel(T* __restrict__ out, float* __restrict__ sum_out, const float* __restrict__ x,
                                        const float* __restrict__ coeff, const T* __restrict__ w, const int* __restrict__ rows, int S,
                                        int W, float eps) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  const float* xr = x + r * S * W;
  float a[NS_MAX_STREAMS];
  for (int s = 0; s < S; ++s) a[s] = coeff[s];
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(a[s], xr[(size_t)s * W + c], u);
    ss = fmaf(u, u, ss);
  }
  ss = block_sum(ss, scratch);
  const float rinv = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(a[s], xr[(size_t)s * W + c], u);
    if (sum_out) sum_out[(size_t)i * W + c] = u;
    if (out) out[(size_t)i * W + c] = from_f<T>(u * rinv * to_f(w[c]));
  }
}

extern "C" int ns_stream_read_norm(void* out, float* sum_out, const float* x, const float* coeff, const void* w, const int* rows,
                                   int n, int S, int W, float eps, int dtype, hipStream_t stream) {
  if (n <= 0 || S <= 0 || S > NS_MAX_STREAMS || W <= 0) return NS_ERR_BAD_ARG;
  const int threads = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  if (dtype == NS_DTYPE_F32)
    stream_read_norm_kernel<float><<<n, threads, 0, stream>>>((float*)out, sum_out, x, coeff, (const float*)w, rows, S, W, eps);
  else if (dtype == NS_DTYPE_BF16)
    stream_read_norm_kernel<bf16_t><<<n, threads, 0, stream>>>((bf16_t*)out, sum_out, x, coeff, (const bf16_t*)w, rows, S, W, eps);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// In place: a thread owns a column of a row, reads its S old values, then writes the S new ones.
template <typename T>
__global__ void stream_write_kernel(float* __restrict__ x, const float* __restrict__ mix, const float* __restrict__ gain,
                                    const T* __restrict__ y, int y_stride, int S, int W) {
  __shared__ float m_s[NS_MAX_STREAMS * NS_MAX_STREAMS + NS_MAX_STREAMS];
  for (int i = threadIdx.x; i < S * S + S; i += blockDim.x) m_s[i] = i < S * S ? mix[i] : gain[i - S * S];
  __syncthreads();
  const size_t r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  float* xr = x + r * S * W + c;
  float old[NS_MAX_STREAMS];
  for (int s = 0; s < S; ++s) old[s] = xr[(size_t)s * W];
  const float yv = to_f(y[r * y_stride + c]);
  for (int t = 0; t < S; ++t) {
    float v = 0.f;
    for (int s = 0; s < S; ++s) v = fmaf(m_s[s * S + t], old[s], v);
    xr[(size_t)t * W] = fmaf(m_s[S * S + t], yv, v);
  }
}

extern "C" int ns_stream_write(float* x, const float* mix, const float* gain, const void* y, int y_stride, int n, int S, int W,
                               int dtype, hipStream_t stream) {
  if (n <= 0 || S <= 0 || S > NS_MAX_STREAMS || W <= 0 || (W + 255) / 256 > 65535) return NS_ERR_BAD_ARG;
  dim3 grid(n, (W + 255) / 256);
  if (dtype == NS_DTYPE_F32)
    stream_write_kernel<float><<<grid, 256, 0, stream>>>(x, mix, gain, (const float*)y, y_stride, S, W);
  else if (dtype == NS_DTYPE_BF16)
    stream_write_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, mix, gain, (const bf16_t*)y, y_stride, S, W);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// out = act(x), element by element; act 0: the tanh form of GELU, 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))); 1: SiLU
template <typename T>
__global__ void activation_kernel(T* __restrict__ out, const T* __restrict__ x, size_t count, int act) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
    const float z = to_f(x[i]);
    float v;
    if (act == 0)
      v = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    else
      v = z / (1.f + expf(-z));
    out[i] = from_f<T>(v);
  }
}

extern "C" int ns_activation(void* out, const void* x, size_t count, int act, int dtype, hipStream_t stream) {
  if (count == 0 || act < 0 || act > 1) return NS_ERR_BAD_ARG;
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    activation_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)x, count, act);
  else if (dtype == NS_DTYPE_BF16)
    activation_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, count, act);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
