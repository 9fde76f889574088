// What lies between an attention layer's input projections and its attention kernel, for layers
// that norm before they rotate: an optional short causal convolution over time on every channel
// of q, k and v, an RMS norm of q and of k with learned weights (per head, one weight vector
// shared by the heads; or over the whole projection, one weight per channel), rotary positions on
// the first r elements of every head (pairs interleaved or split in halves, cos and sin times a
// magnitude), and the write of keys and values into the paged cache.  Values may be the keys as
// they were before norm and rotation (a layer without a value projection).  Further options: a bias
// per projected channel (float, added to the row as it is gathered; not together with a
// convolution), a query temperature 1 + c ln(floor((p + 1) / f) + 1) on q, and heads that hold
// several score maps side by side (`maps`): norm weights and cache rows stay per head, the rotation
// works on each map's own leading elements, and the queries leave expanded, one row of the head's
// width per (head, map) with that map's elements in their place and zeros elsewhere, so that an
// attention kernel over keys of the head's width computes each map's scores on its own.
//
// One block per token, or, in steps of few tokens, one per (token, kv head): the block then takes
// that kv head's key and value and the query heads that read it, so that a decode step still fills
// the chip (what a row's sums are made of and their order do not depend on the split).  The token's
// row is gathered into LDS as floats (the convolution reads up to taps - 1 earlier rows: of this
// step where the entry has them, otherwise the tail that the request's state slot carries), the
// sums of squares are taken in an order that depends on the row alone, and everything after the
// projection is float arithmetic rounded once, on the way out.
#include "common.h"

constexpr int kPrepThreads = 256;
constexpr int kPrepMaxTaps = 8;
constexpr int kPrepSplitTokens = 64;  // up to so many tokens a step, a token's heads are spread over nkv blocks
constexpr int kPrepMaxHeads = 1024;   // q heads + kv heads whose inverse norms are kept in LDS

enum : int { NORM_NONE = 0, NORM_PER_HEAD = 1, NORM_WHOLE = 2 };

struct PrepArgs {
  const void* proj;        // [T, stride]
  int stride, q_off, k_off, v_off;   // v_off < 0: the values are the keys before norm and rotation
  int nh, nkv, hd, vd;
  const float* conv_w;     // [q + k + v channels, taps] or null
  int taps;
  float* tail;             // [slots, taps - 1, channels]: the last projected rows of each request
  const int* state_slots;  // [entries]
  const int* entry_of_token;
  const int* cu_tokens;
  const int* positions;
  int norm_mode;
  const float* q_norm_w;   // [hd] or [nh * hd]
  const float* k_norm_w;   // [hd] or [nkv * hd]
  float eps;
  const float* inv_freq;   // [rotary_dim / 2] or null
  int rotary_dim, half_split;
  float magnitude;
  void* q_out;             // [T, nh * hd]
  void* k_cache;           // [pages, nkv, page_size, hd]
  void* v_cache;           // [pages, nkv, vd, page_size]
  const int* slot_mapping; // [T], -1: store nothing
  int page_size;
  int parts;               // blocks a token: 1, or nkv (a kv head and its query heads each)
  const float* bias;       // [q + k + v channels] or null
  int temp_on;             // query temperature
  float temp_floor, temp_scale;
  int maps;                // score maps a head (1: the plain layout of q_out; > 1: q_out [T, nh * maps * hd], expanded)
  int by8;                 // every offset, stride and width a multiple of 8 (and split halves): eight channels a thread
};

constexpr int kPrepMaxTurns = 256;    // rotary pairs whose cosines and sines a block keeps (a map of up to 512 elements)

template <typename T>
__global__ __launch_bounds__(kPrepThreads) void qk_prep_kernel(PrepArgs a) {
  extern __shared__ __attribute__((aligned(32))) float row[];          // q | k | v of the token, as floats
  __shared__ float red[16];
  __shared__ float inv[kPrepMaxHeads];
  const int t = blockIdx.x;
  // the heads this block takes: all, or kv head blockIdx.y with its query heads
  const int per_kv = a.nh / a.nkv;
  const int qh0 = a.parts > 1 ? blockIdx.y * per_kv : 0, qh1 = a.parts > 1 ? qh0 + per_kv : a.nh;
  const int kh0 = a.parts > 1 ? blockIdx.y : 0, kh1 = a.parts > 1 ? kh0 + 1 : a.nkv;
  const bool every_qk = a.norm_mode == NORM_WHOLE;   // a norm over the whole projection reads all of q and of k
  const int qn = a.nh * a.hd, kn = a.nkv * a.hd;
  const bool own_v = a.v_off >= 0;
  const int vn = own_v ? a.nkv * a.vd : 0;
  const int C = qn + kn + vn;
  const T* proj = (const T*)a.proj;
  const bool all = a.parts == 1;                     // (then no channel or head needs asking)
  auto mine = [&](int c) {
    if (all) return true;
    if (c < qn) return every_qk || (c / a.hd >= qh0 && c / a.hd < qh1);
    if (c < qn + kn) return every_qk || ((c - qn) / a.hd >= kh0 && (c - qn) / a.hd < kh1);
    return (c - qn - kn) / a.vd >= kh0 && (c - qn - kn) / a.vd < kh1;
  };

  // 1. gather, through the convolution where there is one
  if (a.by8) {
    // eight consecutive channels a thread, 16-byte loads (the sums of a channel are those of the scalar form)
    const int e = a.taps > 0 ? a.entry_of_token[t] : 0;
    const int li = a.taps > 0 ? t - a.cu_tokens[e] : 0;
    const float* tail = a.taps > 0 ? a.tail + (size_t)a.state_slots[e] * (a.taps - 1) * C : nullptr;
    for (int c = threadIdx.x * 8; c < C; c += kPrepThreads * 8) {
      if (!mine(c)) continue;
      const int col = c < qn ? a.q_off + c : c < qn + kn ? a.k_off + (c - qn) : a.v_off + (c - qn - kn);
      float y[8];
      if (a.taps > 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = 0.f;
        for (int j = 0; j < a.taps; ++j) {
          const int back = a.taps - 1 - j;
          float u[8];
          if (back <= li) load8(proj + (size_t)(t - back) * a.stride + col, u);
          else load8(tail + (size_t)(a.taps - 1 + li - back) * C + c, u);
#pragma unroll
          for (int i = 0; i < 8; ++i) y[i] = fmaf(a.conv_w[(size_t)(c + i) * a.taps + j], u[i], y[i]);
        }
      } else {
        load8(proj + (size_t)t * a.stride + col, y);
        if (a.bias) {
          float b8[8];
          load8(a.bias + c, b8);
#pragma unroll
          for (int i = 0; i < 8; ++i) y[i] += b8[i];
        }
      }
      store8(row + c, y);
    }
  } else if (a.taps > 0) {
    const int e = a.entry_of_token[t];
    const int li = t - a.cu_tokens[e];                 // the token's place in its entry
    const float* tail = a.tail + (size_t)a.state_slots[e] * (a.taps - 1) * C;
    for (int c = threadIdx.x; c < C; c += kPrepThreads) {
      if (!mine(c)) continue;
      const int col = c < qn ? a.q_off + c : c < qn + kn ? a.k_off + (c - qn) : a.v_off + (c - qn - kn);
      float y = 0.f;
      for (int j = 0; j < a.taps; ++j) {
        const int back = a.taps - 1 - j;               // this tap reads the row `back` tokens ago
        float u;
        if (back <= li) u = to_f32<T>(proj[(size_t)(t - back) * a.stride + col]);
        else u = tail[(size_t)(a.taps - 1 + li - back) * C + c];
        y = fmaf(a.conv_w[(size_t)c * a.taps + j], u, y);
      }
      row[c] = y;
    }
  } else {
    for (int c = threadIdx.x; c < C; c += kPrepThreads) {
      if (!mine(c)) continue;
      const int col = c < qn ? a.q_off + c : c < qn + kn ? a.k_off + (c - qn) : a.v_off + (c - qn - kn);
      const float u = to_f32<T>(proj[(size_t)t * a.stride + col]);
      row[c] = a.bias ? u + a.bias[c] : u;
    }
  }
  __syncthreads();

  // 2. values leave as they are (a layer without a value projection stores its unnormed keys)
  const int slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  if (slot >= 0) {
    const int page = slot / a.page_size, off = slot % a.page_size;
    T* vc = (T*)a.v_cache;
    const float* vsrc = own_v ? row + qn + kn : row + qn;
    for (int i = kh0 * a.vd + threadIdx.x; i < kh1 * a.vd; i += kPrepThreads) {
      const int g = i / a.vd, d = i % a.vd;
      vc[(((size_t)page * a.nkv + g) * a.vd + d) * a.page_size + off] = from_f32<T>(vsrc[i]);
    }
  }

  // 3. inverse norms
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x >> 6;
  const int heads = a.nh + a.nkv;
  if (a.norm_mode == NORM_PER_HEAD) {
    for (int h = wid; h < heads; h += kPrepThreads / kWave) {
      if (!all && !(h < a.nh ? (h >= qh0 && h < qh1) : (h - a.nh >= kh0 && h - a.nh < kh1))) continue;
      const float* x = row + (size_t)h * a.hd;         // (q heads then k heads lie back to back)
      float ss = 0.f;
      for (int d = lane; d < a.hd; d += kWave) ss = fmaf(x[d], x[d], ss);
      ss = wave_sum(ss);
      if (lane == 0) inv[h] = rsqrtf(ss / (float)a.hd + a.eps);
    }
  } else if (a.norm_mode == NORM_WHOLE) {
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < qn; c += kPrepThreads) sq = fmaf(row[c], row[c], sq);
    for (int c = threadIdx.x; c < kn; c += kPrepThreads) sk = fmaf(row[qn + c], row[qn + c], sk);
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    const float iq = rsqrtf(sq / (float)qn + a.eps), ik = rsqrtf(sk / (float)kn + a.eps);
    for (int h = threadIdx.x; h < heads; h += kPrepThreads) inv[h] = h < a.nh ? iq : ik;
  }
  __syncthreads();

  // 4. norm, rotation, and out: a thread takes a pair of a head (or two elements that do not turn)
  const float pos = (float)a.positions[t];
  __shared__ float cs_tab[kPrepMaxTurns], sn_tab[kPrepMaxTurns];      // the token's angles are the same for every head and map
  if (a.inv_freq) {
    for (int i = threadIdx.x; i < a.rotary_dim / 2; i += kPrepThreads) {
      const float ang = pos * a.inv_freq[i];
      cs_tab[i] = cosf(ang) * a.magnitude;
      sn_tab[i] = sinf(ang) * a.magnitude;
    }
    __syncthreads();
  }
  const int sd = a.hd / a.maps;                          // width of one map of a head (the head's, with one map)
  const int half_hd = a.hd / 2, half_sd = sd / 2, half_r = a.rotary_dim / 2;
  T* qo = (T*)a.q_out + (size_t)t * qn * a.maps;
  T* kc = (T*)a.k_cache;
  const float temp = a.temp_on ? 1.0f + a.temp_scale * logf(floorf((pos + 1.0f) / a.temp_floor) + 1.0f) : 1.0f;
  if (a.by8) {
    // Eight consecutive elements a thread, 16-byte stores.  A run in the low half of a map's rotated part comes
    // with its partner run half the rotated width on (the thread turns both); a run behind the rotated part passes.
    const int runs = sd / 8, low = half_r / 8, rot_runs = a.rotary_dim / 8;
    const int per_map = runs - low;                      // work items of a map: low runs (each with its partner) and the rest
    const int page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
    for (int i = threadIdx.x; i < heads * a.maps * per_map; i += kPrepThreads) {
      const int hs = i / per_map, wi = i % per_map;
      const int h = hs / a.maps, mp = hs % a.maps, at = mp * sd;
      if (!all && !(h < a.nh ? (h >= qh0 && h < qh1) : (h - a.nh >= kh0 && h - a.nh < kh1))) continue;
      const bool is_q = h < a.nh, turns = wi < low;
      if (!is_q && slot < 0) continue;
      const int e0 = at + (turns ? wi * 8 : (rot_runs + (wi - low)) * 8);      // first element inside the head
      const int e1 = e0 + half_r;                                               // the partner run (turning runs only)
      float x0[8], x1[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      load8(row + (size_t)h * a.hd + e0, x0);
      if (turns) load8(row + (size_t)h * a.hd + e1, x1);
      if (a.norm_mode != NORM_NONE) {
        const float* w = is_q ? a.q_norm_w : a.k_norm_w;
        const int wbase = a.norm_mode == NORM_WHOLE ? (is_q ? h : h - a.nh) * a.hd : 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          x0[j] = x0[j] * inv[h] * w[wbase + e0 + j];
          if (turns) x1[j] = x1[j] * inv[h] * w[wbase + e1 + j];
        }
      }
      if (turns) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float c = cs_tab[wi * 8 + j], sn = sn_tab[wi * 8 + j];
          const float y0 = x0[j] * c - x1[j] * sn, y1 = x1[j] * c + x0[j] * sn;
          x0[j] = y0;
          x1[j] = y1;
        }
      }
      if (is_q) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          x0[j] *= temp;
          x1[j] *= temp;
        }
        if (a.maps == 1) {
          store8(qo + (size_t)h * a.hd + e0, x0);
          if (turns) store8(qo + (size_t)h * a.hd + e1, x1);
        } else {
          const float zero[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          T* qr = qo + ((size_t)h * a.maps + mp) * a.hd;
          for (int mm = 0; mm < a.maps; ++mm) {
            const int sh = (mm - mp) * sd;
            store8(qr + e0 + sh, mm == mp ? x0 : zero);
            if (turns) store8(qr + e1 + sh, mm == mp ? x1 : zero);
          }
        }
      } else {
        T* kr = kc + (((size_t)page * a.nkv + (h - a.nh)) * a.page_size + off) * a.hd;
        store8(kr + e0, x0);
        if (turns) store8(kr + e1, x1);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < heads * half_hd; i += kPrepThreads) {
    const int hs = i / half_sd, pi = i % half_sd;         // (head, map) and the pair inside the map
    const int h = hs / a.maps, mp = hs % a.maps, at = mp * sd;
    if (!all && !(h < a.nh ? (h >= qh0 && h < qh1) : (h - a.nh >= kh0 && h - a.nh < kh1))) continue;
    int d0, d1;
    bool turns;
    if (pi < half_r) {
      turns = true;
      d0 = a.half_split ? pi : 2 * pi;
      d1 = a.half_split ? pi + half_r : 2 * pi + 1;
    } else {
      turns = false;
      d0 = a.rotary_dim + 2 * (pi - half_r);
      d1 = d0 + 1;
    }
    const bool is_q = h < a.nh;
    d0 += at;
    d1 += at;
    float x0 = row[(size_t)h * a.hd + d0], x1 = row[(size_t)h * a.hd + d1];
    if (a.norm_mode != NORM_NONE) {
      const float* w = is_q ? a.q_norm_w : a.k_norm_w;
      const int wbase = a.norm_mode == NORM_WHOLE ? (is_q ? h : h - a.nh) * a.hd : 0;
      x0 = x0 * inv[h] * w[wbase + d0];
      x1 = x1 * inv[h] * w[wbase + d1];
    }
    if (turns && a.inv_freq) {
      const float c = cs_tab[pi], s = sn_tab[pi];
      const float y0 = x0 * c - x1 * s, y1 = x1 * c + x0 * s;
      x0 = y0;
      x1 = y1;
    }
    if (is_q) {
      x0 *= temp;
      x1 *= temp;
      if (a.maps == 1) {
        qo[(size_t)h * a.hd + d0] = from_f32<T>(x0);
        qo[(size_t)h * a.hd + d1] = from_f32<T>(x1);
      } else {
        // the (head, map)'s own row of the head's width: the map's elements in place, zeros in the other maps' places
        T* qr = qo + ((size_t)h * a.maps + mp) * a.hd;
        for (int mm = 0; mm < a.maps; ++mm) {
          const int sh = (mm - mp) * sd;
          qr[d0 + sh] = from_f32<T>(mm == mp ? x0 : 0.f);
          qr[d1 + sh] = from_f32<T>(mm == mp ? x1 : 0.f);
        }
      }
    } else if (slot >= 0) {
      const int page = slot / a.page_size, off = slot % a.page_size;
      T* kr = kc + (((size_t)page * a.nkv + (h - a.nh)) * a.page_size + off) * a.hd;
      kr[d0] = from_f32<T>(x0);
      kr[d1] = from_f32<T>(x1);
    }
  }
}

// The convolution's tail after a step: the last taps - 1 projected rows of each entry's request
// (rows of this step where the entry brought enough, what the slot held before otherwise).  A
// thread takes one channel of one entry, reads everything it needs and only then writes.
template <typename T>
__global__ void conv_tail_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, int qn, int kn,
                                 int vn, int taps, float* __restrict__ tail, const int* __restrict__ state_slots,
                                 const int* __restrict__ cu_tokens) {
  const int e = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int C = qn + kn + vn;
  if (c >= C) return;
  const int col = c < qn ? q_off + c : c < qn + kn ? k_off + (c - qn) : v_off + (c - qn - kn);
  const int first = cu_tokens[e], len = cu_tokens[e + 1] - first;
  float* mine = tail + (size_t)state_slots[e] * (taps - 1) * C + c;
  float keep[kPrepMaxTaps];
  for (int s = 0; s < taps - 1; ++s) {
    const int li = len - (taps - 1) + s;               // the row that ends up in place s
    keep[s] = li >= 0 ? to_f32<T>(proj[(size_t)(first + li) * stride + col]) : mine[(size_t)(taps - 1 + li) * C];
  }
  for (int s = 0; s < taps - 1; ++s) mine[(size_t)s * C] = keep[s];
}

// proj [T, stride] of `dtype`; q at columns q_off.., k at k_off.., v at v_off.. (v_off < 0: values
// are the unnormed keys, vd must equal hd).  conv_w float [channels, taps] (taps 0: none), tail float
// [slots, taps - 1, channels].  norm_mode 0 none / 1 per head (weights [hd]) / 2 whole projection
// (weights [nh*hd], [nkv*hd]).  inv_freq float [rotary_dim / 2] or null.  Caches K [pages, nkv,
// page_size, hd], V [pages, nkv, vd, page_size]; slot_mapping null or -1: nothing is stored.
// bias float [q + k + v channels] or null (only without a convolution); temp_on: q times
// 1 + temp_scale ln(floor((pos + 1) / temp_floor) + 1); maps > 1: hd is the width of a head's maps
// together, rotary_dim <= hd / maps, and q_out is [T, nh * maps * hd].
SHARPI_EXPORT int sharpi_qk_prep(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off, int n_tokens,
                                 int n_entries, int nh, int nkv, int hd, int vd, const float* conv_w, int taps, float* tail,
                                 const int* state_slots, const int* entry_of_token, const int* cu_tokens,
                                 const int* positions, int norm_mode, const float* q_norm_w, const float* k_norm_w,
                                 float eps, const float* inv_freq, int rotary_dim, int half_split, float magnitude,
                                 void* q_out, void* k_cache, void* v_cache, const int* slot_mapping, int page_size,
                                 int update_tail, const float* bias, int temp_on, float temp_floor, float temp_scale,
                                 int maps, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (maps < 1 || hd % (2 * maps) || rotary_dim > hd / maps) return SHARPI_ERR_ARG;
  if ((bias && taps > 0) || (temp_on && !(temp_floor > 0.f))) return SHARPI_ERR_ARG;
  if (nh <= 0 || nkv <= 0 || hd <= 0 || hd % 2 || vd <= 0 || nh + nkv > kPrepMaxHeads) return SHARPI_ERR_ARG;
  if (taps < 0 || taps == 1 || taps > kPrepMaxTaps || (taps > 0 && (!conv_w || !tail || !state_slots || !cu_tokens || !entry_of_token)))
    return SHARPI_ERR_ARG;
  if (norm_mode < 0 || norm_mode > 2 || (norm_mode && (!q_norm_w || !k_norm_w))) return SHARPI_ERR_ARG;
  if (rotary_dim < 0 || rotary_dim % 2 || rotary_dim > hd || (rotary_dim > 0 && !inv_freq)) return SHARPI_ERR_ARG;
  if (v_off < 0 && vd != hd) return SHARPI_ERR_ARG;
  if (slot_mapping && (!k_cache || !v_cache || page_size <= 0)) return SHARPI_ERR_ARG;
  const int qn = nh * hd, kn = nkv * hd, vn = v_off >= 0 ? nkv * vd : 0;
  const size_t lds = (size_t)(qn + kn + vn) * sizeof(float);
  if (lds > 60 * 1024) return SHARPI_ERR_ARG;
  const int parts = (n_tokens <= kPrepSplitTokens && nkv > 1 && nkv <= 65535 && nh % nkv == 0) ? nkv : 1;
  auto at16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 32 == 0; };
  const int sd = hd / maps;
  const int by8 = (half_split || rotary_dim == 0) && rotary_dim % 16 == 0 && sd % 8 == 0 && vd % 8 == 0 &&
                  stride % 8 == 0 && q_off % 8 == 0 && k_off % 8 == 0 && (v_off < 0 || v_off % 8 == 0) && at16(proj) && at16(q_out) &&
                  at16(k_cache) && at16(tail) && at16(bias) && rotary_dim / 2 <= kPrepMaxTurns;
  if (rotary_dim / 2 > kPrepMaxTurns) return SHARPI_ERR_ARG;
  PrepArgs a{proj, stride, q_off, k_off, v_off, nh, nkv, hd, vd, conv_w, taps, tail, state_slots, entry_of_token,
             cu_tokens, positions, norm_mode, q_norm_w, k_norm_w, eps, rotary_dim > 0 ? inv_freq : nullptr, rotary_dim,
             half_split, magnitude, q_out, k_cache, v_cache, slot_mapping, page_size, parts, bias, temp_on, temp_floor,
             temp_scale, maps, by8};
  dim3 pgrid(n_tokens, parts);
  if (dtype == DT_F32) qk_prep_kernel<float><<<pgrid, kPrepThreads, lds, stream>>>(a);
  else if (dtype == DT_BF16) qk_prep_kernel<bf16_t><<<pgrid, kPrepThreads, lds, stream>>>(a);
  else return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  if (taps > 0 && update_tail) {
    dim3 grid(ceil_div(qn + kn + vn, 256), n_entries);
    if (dtype == DT_F32)
      conv_tail_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, stride, q_off, k_off, v_off, qn, kn, vn, taps,
                                                        tail, state_slots, cu_tokens);
    else
      conv_tail_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)proj, stride, q_off, k_off, v_off, qn, kn, vn, taps,
                                                         tail, state_slots, cu_tokens);
    SHARPI_CHECK_LAUNCH();
  }
  return SHARPI_OK;
}
