// Small row kernels between the products of layers whose branches are gated, summed with scales,
// or fed from the token a second time.
#include "common.h"

// ---------------------------------------------------------------------------
// out [T, N] = x [T, N] * sigmoid(gate), gate = columns g_off.. of proj [T, stride]: the output gate
// of an attention mixer (the heads side by side, gated element by element before the output product).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(const T* __restrict__ x, const T* __restrict__ proj, int stride,
                                                            int g_off, T* __restrict__ out, int n_tokens, int N) {
  const size_t total = (size_t)n_tokens * N;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / N, c = i % N;
    const float z = to_f32<T>(proj[t * stride + g_off + c]);
    out[i] = from_f32<T>(to_f32<T>(x[i]) / (1.0f + expf(-z)));
  }
}

// eight elements a thread, 16-byte accesses (N, stride and g_off multiples of 8)
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate8_kernel(const T* __restrict__ x, const T* __restrict__ proj, int stride,
                                                             int g_off, T* __restrict__ out, int n_tokens, int N) {
  const int per_row = N >> 3;
  const size_t total = (size_t)n_tokens * per_row;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / per_row, c = (i % per_row) << 3;
    float z[8], v[8];
    load8(proj + t * stride + g_off + c, z);
    load8(x + t * N + c, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = v[k] / (1.0f + expf(-z[k]));
    store8(out + t * N + c, v);
  }
}

SHARPI_EXPORT int sharpi_sigmoid_gate(const void* x, const void* proj, int dtype, int stride, int g_off, void* out,
                                      int n_tokens, int N, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (N <= 0 || g_off < 0 || g_off + N > stride) return SHARPI_ERR_ARG;
  const size_t total = (size_t)n_tokens * N;
  const bool by8 = N % 8 == 0 && stride % 8 == 0 && g_off % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 32 == 0 &&
                   reinterpret_cast<uintptr_t>(proj) % 32 == 0 && reinterpret_cast<uintptr_t>(out) % 32 == 0;
  if (by8 && (dtype == DT_F32 || dtype == DT_BF16)) {
    const dim3 block8(256), grid8((unsigned)min((size_t)16384, (total / 8 + 255) / 256));
    if (dtype == DT_F32)
      sigmoid_gate8_kernel<float><<<grid8, block8, 0, stream>>>((const float*)x, (const float*)proj, stride, g_off, (float*)out, n_tokens, N);
    else
      sigmoid_gate8_kernel<bf16_t><<<grid8, block8, 0, stream>>>((const bf16_t*)x, (const bf16_t*)proj, stride, g_off, (bf16_t*)out, n_tokens, N);
    SHARPI_CHECK_LAUNCH();
    return SHARPI_OK;
  }
  const dim3 block(256), grid((unsigned)min((size_t)8192, (total + 255) / 256));
  if (dtype == DT_F32)
    sigmoid_gate_kernel<float><<<grid, block, 0, stream>>>((const float*)x, (const float*)proj, stride, g_off, (float*)out, n_tokens, N);
  else if (dtype == DT_BF16)
    sigmoid_gate_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, (const bf16_t*)proj, stride, g_off, (bf16_t*)out, n_tokens, N);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// The residual sum brought up to date without a norm: h (float) += sum_b s_b x_b (up to 4 branch
// outputs with a scale each, summed in float in the order given), and, with out, the new h in
// out's storage type (what a product behind it reads).
// ---------------------------------------------------------------------------
struct SumArgs {
  const void* x[4];
  float s[4];
};

template <typename TD, typename TO>
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ h, SumArgs a, int n, TO* __restrict__ out,
                                                          size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    float d = 0.f;
    for (int b = 0; b < n; ++b) d = fmaf(a.s[b], to_f32<TD>(((const TD*)a.x[b])[i]), d);
    const float v = h[i] + d;
    h[i] = v;
    if (out) out[i] = from_f32<TO>(v);
  }
}

SHARPI_EXPORT int sharpi_stream_add(float* h, const void* const* xs, const float* scales, int n, int d_dtype, void* out,
                                    int out_dtype, long long total, hipStream_t stream) {
  if (total <= 0) return SHARPI_OK;
  if (n < 0 || n > 4 || (n > 0 && (!xs || !scales))) return SHARPI_ERR_ARG;
  SumArgs a;
  for (int b = 0; b < 4; ++b) {
    a.x[b] = b < n ? xs[b] : nullptr;
    a.s[b] = b < n ? scales[b] : 0.f;
  }
  const dim3 block(256), grid((unsigned)min((size_t)8192, ((size_t)total + 255) / 256));
#define GO(TD, TO) stream_add_kernel<TD, TO><<<grid, block, 0, stream>>>(h, a, n, (TO*)out, (size_t)total)
  if (d_dtype == DT_F32 && (out_dtype == DT_F32 || !out)) GO(float, float);
  else if (d_dtype == DT_F32 && out_dtype == DT_BF16) GO(float, bf16_t);
  else if (d_dtype == DT_BF16 && (out_dtype == DT_BF16 || !out)) GO(bf16_t, bf16_t);
  else if (d_dtype == DT_BF16 && out_dtype == DT_F32) GO(bf16_t, float);
  else return SHARPI_ERR_ARG;
#undef GO
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// out [T, D] = gelu_tanh(gate [T, D]) * table[ids[t], col_off + c]: a layer's slice of a token's row of
// a side table, gated by a product of the stream.
// ---------------------------------------------------------------------------
template <typename T, typename TT>
__global__ __launch_bounds__(256) void side_gate_kernel(const T* __restrict__ gate, const int* __restrict__ ids,
                                                         const TT* __restrict__ table, int table_stride, int col_off,
                                                         T* __restrict__ out, int n_tokens, int D) {
  const size_t total = (size_t)n_tokens * D;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t t = i / D, c = i % D;
    const float g = to_f32<T>(gate[i]);
    const float th = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
    const float e = to_f32<TT>(table[(size_t)ids[t] * table_stride + col_off + c]);
    out[i] = from_f32<T>((0.5f * g * (1.0f + th)) * e);
  }
}

SHARPI_EXPORT int sharpi_side_gate(const void* gate, int dtype, const int* ids, const void* table, int table_dtype,
                                   int table_stride, int col_off, void* out, int n_tokens, int D, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (D <= 0 || col_off < 0 || col_off + D > table_stride) return SHARPI_ERR_ARG;
  const size_t total = (size_t)n_tokens * D;
  const dim3 block(256), grid((unsigned)min((size_t)8192, (total + 255) / 256));
#define GO(T, TT) side_gate_kernel<T, TT><<<grid, block, 0, stream>>>((const T*)gate, ids, (const TT*)table, table_stride, col_off, (T*)out, n_tokens, D)
  if (dtype == DT_F32 && table_dtype == DT_F32) GO(float, float);
  else if (dtype == DT_F32 && table_dtype == DT_BF16) GO(float, bf16_t);
  else if (dtype == DT_BF16 && table_dtype == DT_BF16) GO(bf16_t, bf16_t);
  else if (dtype == DT_BF16 && table_dtype == DT_F32) GO(bf16_t, float);
  else return SHARPI_ERR_ARG;
#undef GO
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
