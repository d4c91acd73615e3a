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

// The two in one pass with 16-byte accesses, for S <= 4 streams and rows of a multiple of four up to 8,192 columns: the
// write of one sublayer's output (``y`` given) followed by the read for the next sublayer (``coeff`` given), each
// optional.  A thread keeps its columns of the mix u in registers between the sum of squares and the output, so a row is
// read once.  ``store`` = 0 leaves x as it was (the last read of a step, whose written streams nobody reads again).
template <typename T, int S, int KMAX>
__global__ __launch_bounds__(256) void stream_step_kernel(float* __restrict__ x, const float* __restrict__ mix, const float* __restrict__ gain,
                                                          const T* __restrict__ y, int y_stride, const float* __restrict__ coeff,
                                                          const T* __restrict__ w, const int* __restrict__ rows, T* __restrict__ out,
                                                          float* __restrict__ sum_out, int W, float eps, int store) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  float* xr = x + r * S * W;
  float m[S][S], gn[S], a[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    gn[s] = y ? gain[s] : 0.f;
    a[s] = coeff ? coeff[s] : 0.f;
#pragma unroll
    for (int t = 0; t < S; ++t) m[s][t] = y ? mix[s * S + t] : (s == t ? 1.f : 0.f);
  }
  float4 u[KMAX];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int c = (threadIdx.x + k * 256) * 4;
    if (c < W) {
      float4 v[S];
#pragma unroll
      for (int s = 0; s < S; ++s) v[s] = *reinterpret_cast<const float4*>(xr + (size_t)s * W + c);
      if (y) {
        const T* yp = y + r * y_stride + c;
        const float4 yv = {to_f(yp[0]), to_f(yp[1]), to_f(yp[2]), to_f(yp[3])};
        float4 nv[S];
#pragma unroll
        for (int t = 0; t < S; ++t) {
          float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < S; ++s) {
            acc.x = fmaf(m[s][t], v[s].x, acc.x), acc.y = fmaf(m[s][t], v[s].y, acc.y);
            acc.z = fmaf(m[s][t], v[s].z, acc.z), acc.w = fmaf(m[s][t], v[s].w, acc.w);
          }
          nv[t] = {fmaf(gn[t], yv.x, acc.x), fmaf(gn[t], yv.y, acc.y), fmaf(gn[t], yv.z, acc.z), fmaf(gn[t], yv.w, acc.w)};
        }
#pragma unroll
        for (int t = 0; t < S; ++t) {
          v[t] = nv[t];
          if (store) *reinterpret_cast<float4*>(xr + (size_t)t * W + c) = nv[t];
        }
      }
      float4 mixv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < S; ++s) {
        mixv.x = fmaf(a[s], v[s].x, mixv.x), mixv.y = fmaf(a[s], v[s].y, mixv.y);
        mixv.z = fmaf(a[s], v[s].z, mixv.z), mixv.w = fmaf(a[s], v[s].w, mixv.w);
      }
      u[k] = mixv;
      ss += mixv.x * mixv.x + mixv.y * mixv.y + mixv.z * mixv.z + mixv.w * mixv.w;
    }
  }
  if (!coeff) return;
  ss = block_sum(ss, scratch);
  const float rinv = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int c = (threadIdx.x + k * 256) * 4;
    if (c < W) {
      if (sum_out) *reinterpret_cast<float4*>(sum_out + (size_t)i * W + c) = u[k];
      if (out) {
        T* op = out + (size_t)i * W + c;
        op[0] = from_f<T>(u[k].x * rinv * to_f(w[c])), op[1] = from_f<T>(u[k].y * rinv * to_f(w[c + 1]));
        op[2] = from_f<T>(u[k].z * rinv * to_f(w[c + 2])), op[3] = from_f<T>(u[k].w * rinv * to_f(w[c + 3]));
      }
    }
  }
}

template <typename T, int S>
static void stream_step_launch(float* x, const float* mix, const float* gain, const void* y, int y_stride, const float* coeff, const void* w,
                               const int* rows, void* out, float* sum_out, int n, int W, float eps, int store, hipStream_t stream) {
  if (W <= 2048)
    stream_step_kernel<T, S, 2><<<n, 256, 0, stream>>>(x, mix, gain, (const T*)y, y_stride, coeff, (const T*)w, rows, (T*)out, sum_out, W, eps, store);
  else
    stream_step_kernel<T, S, 8><<<n, 256, 0, stream>>>(x, mix, gain, (const T*)y, y_stride, coeff, (const T*)w, rows, (T*)out, sum_out, W, eps, store);
}

extern "C" int ns_stream_step(float* x, const float* mix, const float* gain, const void* y, int y_stride, const float* coeff, const void* w,
                              const int* rows, void* out, float* sum_out, int n, int S, int W, float eps, int store, int dtype,
                              hipStream_t stream) {
  if (n <= 0 || S <= 0 || S > 4 || W <= 0 || W > 8192 || W % 4 || (!y && !coeff)) return NS_ERR_BAD_ARG;
  if (y && (!mix || !gain)) return NS_ERR_BAD_ARG;
  if (y && rows && store) return NS_ERR_BAD_ARG;  // a write that is kept covers every row
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
#define NS_STEP(SS)                                                                                                                  \
  if (dtype == NS_DTYPE_F32) stream_step_launch<float, SS>(x, mix, gain, y, y_stride, coeff, w, rows, out, sum_out, n, W, eps, store, stream); \
  else stream_step_launch<bf16_t, SS>(x, mix, gain, y, y_stride, coeff, w, rows, out, sum_out, n, W, eps, store, stream)
  switch (S) {
    case 1: NS_STEP(1); break;
    case 2: NS_STEP(2); break;
    case 3: NS_STEP(3); break;
    default: NS_STEP(4); break;
  }
#undef NS_STEP
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

__device__ __forceinline__ float act_of(float z, int act) {
  return act == 0 ? 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))) : z / (1.f + expf(-z));
}

// The same with 16-byte accesses, for counts that are a multiple of 16 bytes' worth and aligned pointers.
template <typename T>
__global__ void activation_vec_kernel(T* __restrict__ out, const T* __restrict__ x, size_t nvec, int act) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const vec_t* xv = reinterpret_cast<const vec_t*>(x);
  vec_t* ov = reinterpret_cast<vec_t*>(out);
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (size_t)gridDim.x * blockDim.x) {
    const vec_t a = xv[i];
    vec_t r;
#pragma unroll
    for (int e = 0; e < V; ++e) r[e] = from_f<T>(act_of(to_f(a[e]), act));
    ov[i] = r;
  }
}

extern "C" int ns_activation(void* out, const void* x, size_t count, int act, int dtype, hipStream_t stream) {
  if (count == 0 || act < 0 || act > 1) return NS_ERR_BAD_ARG;
  if (dtype != NS_DTYPE_F32 && dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
  const size_t per = dtype == NS_DTYPE_F32 ? 4 : 8;
  if (count % per == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)x % 16) == 0) {
    const size_t nvec = count / per;
    size_t blocks = (nvec + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (dtype == NS_DTYPE_F32)
      activation_vec_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)x, nvec, act);
    else
      activation_vec_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, nvec, act);
    return ns_launch_status();
  }
  size_t blocks = (count + 255) / 256;
  if (blocks > 65535) blocks = 65535;
  if (dtype == NS_DTYPE_F32)
    activation_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)out, (const float*)x, count, act);
  else
    activation_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, count, act);
  return ns_launch_status();
}
