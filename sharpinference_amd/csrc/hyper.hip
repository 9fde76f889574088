// Several residual streams in place of one (hyper-connections).
//
// A token carries S float rows x_0 .. x_(S-1) of the model's width, kept [token][stream][width].  A
// sublayer reads u = sum_s in[s] x_s, and its output y comes back into every stream at once:
// x_t <- sum_s mix[s][t] x_s + out[t] y, all from the old rows.  One kernel does what lies between two
// sublayers: it brings the streams up to date with the output still waiting (if there is one), stores
// them, forms the next sublayer's u and normalises it (RMS norm with a weight), one block a token.
// The same kernel closes the model: with no read weights u is the plain sum of the streams, and
// without a norm it is stored as it is, in float.  The first sublayer of a model finds its streams
// all equal to one row (a stride of zero between the streams of the source).
//
// The waiting output may be a tensor, or the routed feed-forward's sum still to be formed: rows
// pos[r k .. r k + k) of y, each times its weight, plus the shared expert's row, added in that order in
// float and rounded once to the storage type (what a separate combine kernel would have stored).
// Everything else is float: the streams, the mixing, the statistics.
#include "common.h"

constexpr int kHyperThreads = 256;
constexpr int kHyperMaxStreams = 8;

struct HyperArgs {
  const float* src;        // the old streams: element (r, s, c) at r * src_token + s * src_stream + c
  long long src_token, src_stream;
  float* lanes;            // [T, S, W]: the new streams are stored here (null: not stored)
  const void* delta;       // [T, W] the waiting output, or the experts' rows; null: nothing waits
  const int* sum_pos;      // expert sum: [T * k] rows of delta; null: delta is the output itself
  const void* sum_shared;  // [T, W] or null
  const float* sum_w;      // [T * k] or null (ones)
  int sum_k;
  const float* mix;        // [S, S] (from, to); with delta
  const float* outw;       // [S]; with delta
  const float* inw;        // [S] or null (ones)
  const void* norm_w;      // [W] or null: u is stored unnormalised, as float
  float eps;
  void* out;               // [rows, W] (norm_w: the output's type; else float)
  const int* rows;         // the tokens to produce, or null: all
  int S, W;
};

template <typename TD, int V>
__device__ __forceinline__ void hyper_delta(const HyperArgs& a, int r, int c, float* d) {
  const TD* delta = (const TD*)a.delta;
  if (!a.sum_pos) {
    if (V == 8) load8(delta + (size_t)r * a.W + c, d);
    else d[0] = to_f32<TD>(delta[(size_t)r * a.W + c]);
    return;
  }
#pragma unroll
  for (int j = 0; j < V; ++j) d[j] = 0.f;
  for (int q = 0; q < a.sum_k; ++q) {
    float v[V];
    const TD* row = delta + (size_t)a.sum_pos[r * a.sum_k + q] * a.W + c;
    if (V == 8) load8(row, v);
    else v[0] = to_f32<TD>(row[0]);
    const float wq = a.sum_w ? a.sum_w[r * a.sum_k + q] : 1.0f;
#pragma unroll
    for (int j = 0; j < V; ++j) d[j] += a.sum_w ? wq * v[j] : v[j];
  }
  if (a.sum_shared) {
    float v[V];
    const TD* row = (const TD*)a.sum_shared + (size_t)r * a.W + c;
    if (V == 8) load8(row, v);
    else v[0] = to_f32<TD>(row[0]);
#pragma unroll
    for (int j = 0; j < V; ++j) d[j] += v[j];
  }
#pragma unroll
  for (int j = 0; j < V; ++j) d[j] = to_f32<TD>(from_f32<TD>(d[j]));
}

template <typename TD, typename TW, typename TO, int S, int V>
__global__ __launch_bounds__(kHyperThreads) void hyper_step_kernel(HyperArgs a) {
  extern __shared__ float u_row[];          // the sublayer's input row, between the two passes
  __shared__ float red[16];
  __shared__ float cm[S * S], co[S], ci[S];
  const int i = blockIdx.x;
  const int r = a.rows ? a.rows[i] : i;
  if (threadIdx.x < S * S) cm[threadIdx.x] = a.mix ? a.mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    co[threadIdx.x] = a.outw ? a.outw[threadIdx.x] : 0.f;
    ci[threadIdx.x] = a.inw ? a.inw[threadIdx.x] : 1.0f;
  }
  __syncthreads();
  const float* src = a.src + (size_t)r * a.src_token;
  const bool waits = a.delta != nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x * V; c < a.W; c += kHyperThreads * V) {
    float x[S][V];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if (V == 8) load8(src + (size_t)s * a.src_stream + c, x[s]);
      else x[s][0] = src[(size_t)s * a.src_stream + c];
    }
    float u[V];
#pragma unroll
    for (int j = 0; j < V; ++j) u[j] = 0.f;
    if (waits) {
      float d[V];
      hyper_delta<TD, V>(a, r, c, d);
#pragma unroll
      for (int t = 0; t < S; ++t) {
        float nx[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < S; ++s) acc = fmaf(cm[s * S + t], x[s][j], acc);
          nx[j] = fmaf(co[t], d[j], acc);
          u[j] = fmaf(ci[t], nx[j], u[j]);
        }
        if (a.lanes) {
          float* dst = a.lanes + ((size_t)r * S + t) * a.W + c;
          if (V == 8) store8(dst, nx);
          else dst[0] = nx[0];
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < S; ++t) {
#pragma unroll
        for (int j = 0; j < V; ++j) u[j] = fmaf(ci[t], x[t][j], u[j]);
        if (a.lanes && a.lanes != a.src) {
          float* dst = a.lanes + ((size_t)r * S + t) * a.W + c;
          if (V == 8) store8(dst, x[t]);
          else dst[0] = x[t][0];
        }
      }
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      u_row[c + j] = u[j];
      ss = fmaf(u[j], u[j], ss);
    }
  }
  if (!a.norm_w) {                            // the closing sum: stored as it is
    __syncthreads();
    float* o = (float*)a.out + (size_t)i * a.W;
    for (int c = threadIdx.x; c < a.W; c += kHyperThreads) o[c] = u_row[c];
    return;
  }
  const float total = block_sum(ss, red);     // (its barriers also make the row visible)
  const float sc = 1.0f / sqrtf(total / (float)a.W + a.eps);
  const TW* w = (const TW*)a.norm_w;
  TO* o = (TO*)a.out + (size_t)i * a.W;
  for (int c = threadIdx.x * V; c < a.W; c += kHyperThreads * V) {
    if (V == 8) {
      float wv[8], y[8];
      load8(w + c, wv);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (u_row[c + j] * sc) * wv[j];
      store8(o + c, y);
    } else {
      o[c] = from_f32<TO>((u_row[c] * sc) * to_f32<TW>(w[c]));
    }
  }
}

template <typename TD, typename TW, typename TO, int V>
static int hyper_launch_s(const HyperArgs& a, int n_rows, hipStream_t stream) {
  const size_t lds = (size_t)a.W * sizeof(float);
#define HYPER_S(SV)                                                                                 \
  case SV:                                                                                          \
    hyper_step_kernel<TD, TW, TO, SV, V><<<n_rows, kHyperThreads, lds, stream>>>(a);                \
    break
  switch (a.S) {
    HYPER_S(1); HYPER_S(2); HYPER_S(3); HYPER_S(4); HYPER_S(5); HYPER_S(6); HYPER_S(7); HYPER_S(8);
    default: return SHARPI_ERR_ARG;
  }
#undef HYPER_S
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

template <typename TD, typename TW, typename TO>
static int hyper_launch_v(const HyperArgs& a, int n_rows, bool by8, hipStream_t stream) {
  return by8 ? hyper_launch_s<TD, TW, TO, 8>(a, n_rows, stream) : hyper_launch_s<TD, TW, TO, 1>(a, n_rows, stream);
}

// src float: the old streams, element (token r, stream s, column c) at r * src_token + s * src_stream + c
// (src_stream 0: every stream is the one row).  lanes float [T, S, W] or null.  delta (delta_dtype)
// [T, W], or with sum_pos int [T * k] the experts' rows (+ sum_shared [T, W], sum_w float [T * k], both
// optional); null: nothing waits.  mix float [S, S], outw float [S] (with delta), inw float [S] or null (ones).
// norm_w (w_dtype) [W] with eps: out (out_dtype) [n_rows, W] = the normalised u; norm_w null: out float
// [n_rows, W] = u.  rows int [n_rows] or null (n_rows = T: all tokens, in order).
SHARPI_EXPORT int sharpi_hyper_step(const float* src, long long src_token, long long src_stream, float* lanes,
                                    const void* delta, int delta_dtype, const int* sum_pos, const void* sum_shared,
                                    const float* sum_w, int sum_k, const float* mix, const float* outw, const float* inw,
                                    const void* norm_w, int w_dtype, float eps, void* out, int out_dtype, const int* rows,
                                    int n_rows, int S, int W, hipStream_t stream) {
  if (n_rows <= 0) return SHARPI_OK;
  if (!src || !out || S < 1 || S > kHyperMaxStreams || W <= 0 || (size_t)W * sizeof(float) > 60 * 1024) return SHARPI_ERR_ARG;
  if (delta && (!mix || !outw)) return SHARPI_ERR_ARG;
  if (sum_pos && (!delta || sum_k <= 0)) return SHARPI_ERR_ARG;
  if (!norm_w) out_dtype = DT_F32;
  const HyperArgs a{src, src_token, src_stream, lanes, delta, sum_pos, sum_shared, sum_w, sum_k, mix, outw, inw, norm_w, eps,
                    out, rows, S, W};
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 32 == 0; };
  const bool by8 = W % 8 == 0 && src_token % 8 == 0 && src_stream % 8 == 0 && aligned(src) && aligned(lanes) && aligned(delta) &&
                   aligned(sum_shared) && aligned(norm_w) && aligned(out);
  if (delta_dtype != DT_F32 && delta_dtype != DT_BF16) return SHARPI_ERR_ARG;
#define HYPER_GO(TD)                                                                                        \
  do {                                                                                                      \
    if (!norm_w || (w_dtype == DT_F32 && out_dtype == DT_F32)) return hyper_launch_v<TD, float, float>(a, n_rows, by8, stream); \
    if (w_dtype == DT_F32 && out_dtype == DT_BF16) return hyper_launch_v<TD, float, bf16_t>(a, n_rows, by8, stream);   \
    if (w_dtype == DT_BF16 && out_dtype == DT_BF16) return hyper_launch_v<TD, bf16_t, bf16_t>(a, n_rows, by8, stream); \
    if (w_dtype == DT_BF16 && out_dtype == DT_F32) return hyper_launch_v<TD, bf16_t, float>(a, n_rows, by8, stream);   \
  } while (0)
  if (delta_dtype == DT_F32) HYPER_GO(float);
  else HYPER_GO(bf16_t);
#undef HYPER_GO
  return SHARPI_ERR_ARG;
}

// ---------------------------------------------------------------------------
// The difference of two score maps: a [T, H, 2, e] holds per head the outputs a1, a2 of two attentions
// over the same values; out [T, H, e] = unit_rms(a1 - lambda a2) * post * gate, the root mean square over the
// head's e values in float (eps inside the root), gate = sigmoid(z) with z column g_off + h of proj
// [T, stride] (one number per head; proj null: no gate).  A wave a (token, head).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void map_difference_kernel(const T* __restrict__ a, float lambda, float eps, float post,
                                                             const T* __restrict__ proj, int stride, int g_off,
                                                             T* __restrict__ out, int n_pairs, int H, int e) {
  const int lane = threadIdx.x & (kWave - 1);
  const int p = blockIdx.x * (256 / kWave) + (threadIdx.x >> 6);       // (token, head)
  if (p >= n_pairs) return;
  const T* a1 = a + (size_t)p * 2 * e;
  const T* a2 = a1 + e;
  float ss = 0.f;
  for (int c = lane; c < e; c += kWave) {
    const float d = to_f32<T>(a1[c]) - lambda * to_f32<T>(a2[c]);
    ss = fmaf(d, d, ss);
  }
  ss = wave_sum(ss);
  float mul = post / sqrtf(ss / (float)e + eps);
  if (proj) {
    const int t = p / H, h = p % H;
    const float z = to_f32<T>(proj[(size_t)t * stride + g_off + h]);
    mul *= 1.0f / (1.0f + expf(-z));
  }
  T* o = out + (size_t)p * e;
  for (int c = lane; c < e; c += kWave) {
    const float d = to_f32<T>(a1[c]) - lambda * to_f32<T>(a2[c]);
    o[c] = from_f32<T>(d * mul);
  }
}

SHARPI_EXPORT int sharpi_map_difference(const void* a, int dtype, float lambda, float eps, float post, const void* proj,
                                        int stride, int g_off, void* out, int n_tokens, int H, int e, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (H <= 0 || e <= 0 || (proj && (g_off < 0 || g_off + H > stride))) return SHARPI_ERR_ARG;
  const long long pairs = (long long)n_tokens * H;
  if (pairs > 0x7fffffffLL) return SHARPI_ERR_ARG;
  const dim3 block(256), grid((unsigned)((pairs + 3) / 4));
  if (dtype == DT_F32)
    map_difference_kernel<float><<<grid, block, 0, stream>>>((const float*)a, lambda, eps, post, (const float*)proj, stride, g_off,
                                                             (float*)out, (int)pairs, H, e);
  else if (dtype == DT_BF16)
    map_difference_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)a, lambda, eps, post, (const bf16_t*)proj, stride,
                                                              g_off, (bf16_t*)out, (int)pairs, H, e);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
