// Matrix-valued recurrent states with one scalar decay per (token, head), walked token by token.
//
// Per head a state S [dk, dv] (float) moves as S_t = a_t S_(t-1) + b_t k_t v_t^T and gives o_t = S_t^T q_t.
// Two designs of mixer share the walk; they differ in where a_t and b_t come from and in what is done
// with o_t:
//   WALK_EXP_GATES  (a matrix memory with exponential gates): from pre-activations x_i, x_f of a token's
//       head, i = cap tanh((x_i + bias_i) / cap), f = log_sigmoid(cap tanh((x_f + bias_f) / cap)), a running
//       maximum m_t = max(f + m_(t-1), i) (m starts at 0), a_t = exp(f + m_(t-1) - m_t), b_t = exp(i - m_t);
//       beside S a vector n_t = a_t n_(t-1) + b_t k_t; the output is o_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
//   WALK_STATE_SPACE (a selective state space): dt = softplus(x_dt + bias_dt), a_t = exp(-exp(A_log) dt),
//       b_t = dt; k and q are the state's input and output vectors, shared by the heads of a group; the
//       output is o_t + D v_t.
//   WALK_FIXED_DECAY (retention): a_t is one stored number per head and b_t one number for the layer (the
//       keys' scale); q and k are first turned by rotary positions on their leading elements (pairs (i, i +
//       r/2), angle = position x frequency, in float, on the staged floats), the output is o_t itself.
// Everything but the reading of q, k, v is float: the gates, their logarithms and exponentials, the
// running maximum, the state, the sums.
//
// Work: a block (one wave) = (entry, head, 8 value columns).  Lane (g, j) keeps RPL = DKP / 8 rows
// g RPL .. g RPL + RPL - 1 of column j in registers (DKP = dk rounded up to 32, 64, 128 or 256; rows
// beyond dk stay zero).  Tokens are staged 8 at a time into LDS (8 KB a block at 128 rows: with 16 a
// CU held ten waves and the walk took 1.4 times as long; with 4 the gates' arithmetic, done once a
// stage, weighs more): q and k as floats in the order the
// lanes read them, the stage's gates computed side by side (the running maximum by a scan over
// the lanes whose order is fixed by the chunk), then the wave walks the stage's tokens.  A request's
// state lies slice by slice, [heads, ceil(dv / 8), slice], a slice = RPL x 64 floats of S in the
// lanes' order (row g RPL + r of column j at r 64 + 8 g + j), and, for the exponential gates, DKP
// floats of n and the maximum m (each slice its own copy: the blocks of a head do not wait for
// each other).
//
// A long entry alone in its step would leave most of the chip idle.  Since a_t is one number per head,
// a stretch of tokens acts on the state as S -> D S + L with D the product of its decays and L what
// the stretch makes of a zero state, so the entry is cut into segments that are walked side by side:
// WALK_LOCAL walks every segment but an entry's last from nothing (for the exponential gates the
// maximum starts at minus infinity: the first token then enters with weight 1) and keeps L, its
// maximum and the summed logarithms of the decays; a short kernel turns these into the segments' true
// start states one after the other (for the gates, with m' = max(F + m, m_L):
// S' = exp(F + m - m') S + exp(m_L - m') L); WALK_FINAL walks every segment from its start state,
// writes the outputs, and the entry's last segment leaves the new state in the slot.
#include "common.h"

enum : int { WALK_EXP_GATES = 0, WALK_STATE_SPACE = 1, WALK_FIXED_DECAY = 2 };
enum : int { WALK_WHOLE = 0, WALK_LOCAL = 1, WALK_FINAL = 2 };
constexpr int kWalkCols = 8;       // value columns of a block
constexpr int kWalkChunk = 8;      // tokens staged at a time
constexpr float kWalkFloor = 1e-6f;

SHARPI_EXPORT int sharpi_state_walk_cols() { return kWalkCols; }

// floats of a slice: S, then (exponential gates) n and 8 floats that begin with m
static inline __host__ __device__ int walk_slice_floats(int dkp, int mode) {
  return (dkp / 8) * 64 + (mode == WALK_EXP_GATES ? dkp + 8 : 0);
}
SHARPI_EXPORT int sharpi_state_walk_slice_floats(int dk, int mode) {
  const int dkp = dk <= 32 ? 32 : dk <= 64 ? 64 : dk <= 128 ? 128 : 256;
  return walk_slice_floats(dkp, mode);
}

__device__ __forceinline__ float softplus_f32(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float log_sigmoid_f32(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// 16 bytes of a row as floats
__device__ __forceinline__ void load16(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
__device__ __forceinline__ void load16(const bf16_t* p, float* v) { load8(p, v); }

// where row `row` (= g RPL + r) of a staged q or k vector lies in LDS: four rows of a lane together,
// the eight row groups side by side (a lane reads float4s, the wave 32 consecutive words)
template <int RPL>
__device__ __forceinline__ int staged_at(int row) {
  const int g = row / RPL, r = row % RPL;
  return ((r >> 2) * 8 + g) * 4 + (r & 3);
}

template <typename T, int RPL, int MODE, int PHASE>
__global__ __launch_bounds__(kWave) void state_walk_kernel(
    const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off, int heads_per_group,
    const float* __restrict__ gates, int gate_stride, const float* __restrict__ p0, const float* __restrict__ p1,
    const float* __restrict__ p2, float cap, float q_scale, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_tokens, float* __restrict__ out, int nh, int dk,
    int dv, int ncb, int vec, const int* __restrict__ segs, float* __restrict__ seg_local,
    const float* __restrict__ seg_start, float* __restrict__ seg_decay, const int* __restrict__ positions,
    const float* __restrict__ inv_freq, int rot_dim, float k_scale) {
  constexpr int DKP = RPL * 8;
  constexpr int V = 16 / (int)sizeof(T);            // elements of a 16-byte load
  __shared__ __attribute__((aligned(16))) float q_s[PHASE == WALK_LOCAL ? 1 : kWalkChunk][DKP];     // (no outputs, no queries)
  __shared__ __attribute__((aligned(16))) float k_s[kWalkChunk][DKP];
  __shared__ float v_s[kWalkChunk][kWalkCols];
  __shared__ float a_s[kWalkChunk], b_s[kWalkChunk], e_s[kWalkChunk];
  const int cb = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x, g = lane >> 3, j = lane & 7;
  const int slice = walk_slice_floats(DKP, MODE);
  int e, t_first, t_end;
  bool last = true;
  if (PHASE == WALK_WHOLE) {
    e = blockIdx.z;
    t_first = cu_tokens[e];
    t_end = cu_tokens[e + 1];
  } else {
    const int* sg = segs + 4 * blockIdx.z;
    e = sg[0];
    t_first = sg[1];
    t_end = t_first + sg[2];
    last = sg[3] != 0;
    if (PHASE == WALK_LOCAL && last) return;        // nobody starts from what an entry's last segment makes
  }
  if (t_end <= t_first) return;
  const size_t seg_at = (((size_t)blockIdx.z * nh + h) * ncb + cb) * slice;
  float* st = state + (((size_t)state_slots[e] * nh + h) * ncb + cb) * slice;      // the request's slot
  const float* from = PHASE == WALK_FINAL ? seg_start + seg_at : st;
  const int c = cb * kWalkCols + j;
  const int qk_head = h / heads_per_group;

  float S[RPL], n[RPL];
  float m_run = 0.f, log_decay = 0.f;
  if (PHASE == WALK_LOCAL) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) S[r] = 0.f, n[r] = 0.f;
    m_run = -INFINITY;
  } else {
#pragma unroll
    for (int r = 0; r < RPL; ++r) S[r] = from[r * 64 + lane];
    if (MODE == WALK_EXP_GATES) {
      const float4* nsrc = reinterpret_cast<const float4*>(from + RPL * 64);
#pragma unroll
      for (int r4 = 0; r4 < RPL / 4; ++r4) {
        const float4 x = nsrc[r4 * 8 + g];
        n[r4 * 4] = x.x; n[r4 * 4 + 1] = x.y; n[r4 * 4 + 2] = x.z; n[r4 * 4 + 3] = x.w;
      }
      m_run = from[RPL * 64 + DKP];
    }
  }
  float par0 = 0.f, par1 = 0.f, par2 = 0.f;     // the head's constants
  if (MODE == WALK_EXP_GATES) {
    par0 = p0[h];
    par1 = p1[h];
  } else if (MODE == WALK_FIXED_DECAY) {
    par0 = p0[h];                 // the head's decay
    par1 = logf(par0);
  } else {
    par0 = p0[h];                 // dt bias
    par1 = -expf(p1[h]);          // -exp(A_log)
    par2 = p2[h];                 // D
  }

  for (int t0 = t_first; t0 < t_end; t0 += kWalkChunk) {
    const int nt = min(kWalkChunk, t_end - t0);
    __syncthreads();
    // stage q and k (floats, the lanes' order), v, and the tokens' gates
    if (vec) {                                       // 16-byte loads: every head's q and k begin on a 16-byte border
      constexpr int VPR = DKP / V;                   // loads of a row
      for (int idx = lane; idx < kWalkChunk * VPR; idx += kWave) {
        const int tt = idx / VPR, row0 = (idx % VPR) * V;
        float qv[V], kv[V];
#pragma unroll
        for (int i = 0; i < V; ++i) qv[i] = 0.f, kv[i] = 0.f;
        if (tt < nt && row0 < dk) {
          const T* base = proj + (size_t)(t0 + tt) * stride + (size_t)qk_head * dk + row0;
          load16(base + q_off, qv);
          load16(base + k_off, kv);
        }
#pragma unroll
        for (int i = 0; i < V; i += 4) {             // four rows of a lane lie together
          const int at = staged_at<RPL>(row0 + i);
          if (PHASE != WALK_LOCAL) *reinterpret_cast<float4*>(&q_s[tt][at]) = make_float4(qv[i] * q_scale, qv[i + 1] * q_scale, qv[i + 2] * q_scale, qv[i + 3] * q_scale);
          *reinterpret_cast<float4*>(&k_s[tt][at]) = make_float4(kv[i], kv[i + 1], kv[i + 2], kv[i + 3]);
        }
      }
    } else
    for (int idx = lane; idx < kWalkChunk * DKP; idx += kWave) {
      const int tt = idx / DKP, row = idx % DKP;
      float qv = 0.f, kv = 0.f;
      if (tt < nt && row < dk) {
        const T* base = proj + (size_t)(t0 + tt) * stride + (size_t)qk_head * dk + row;
        qv = to_f32<T>(base[q_off]) * q_scale;
        kv = to_f32<T>(base[k_off]);
      }
      const int at = staged_at<RPL>(row);
      if (PHASE != WALK_LOCAL) q_s[tt][at] = qv;
      k_s[tt][at] = kv;
    }
    for (int idx = lane; idx < kWalkChunk * kWalkCols; idx += kWave) {
      const int tt = idx / kWalkCols, jj = idx % kWalkCols;
      const int cc = cb * kWalkCols + jj;
      v_s[tt][jj] = (tt < nt && cc < dv) ? to_f32<T>(proj[(size_t)(t0 + tt) * stride + v_off + (size_t)h * dv + cc]) : 0.f;
    }
    if (MODE == WALK_FIXED_DECAY) {
      if (lane < nt) {
        a_s[lane] = par0;
        b_s[lane] = k_scale;
      }
      if (PHASE == WALK_LOCAL) log_decay += (float)nt * par1;
      if (rot_dim > 0) {
        // rotary positions on the staged floats: element i of a head with element i + rot_dim / 2
        __syncthreads();
        const int half = rot_dim >> 1;
        for (int idx = lane; idx < nt * half; idx += kWave) {
          const int tt = idx / half, i = idx % half;
          const float ang = (float)positions[t0 + tt] * inv_freq[i];
          const float cs = cosf(ang), sn = sinf(ang);
          const int at0 = staged_at<RPL>(i), at1 = staged_at<RPL>(i + half);
          const float ku = k_s[tt][at0], kv = k_s[tt][at1];
          k_s[tt][at0] = ku * cs - kv * sn;
          k_s[tt][at1] = kv * cs + ku * sn;
          if (PHASE != WALK_LOCAL) {
            const float qu = q_s[tt][at0], qv = q_s[tt][at1];
            q_s[tt][at0] = qu * cs - qv * sn;
            q_s[tt][at1] = qv * cs + qu * sn;
          }
        }
      }
    } else {
      const bool live = lane < nt;
      const float* grow = gates + (size_t)(t0 + (live ? lane : 0)) * gate_stride;
      if (MODE == WALK_EXP_GATES) {
        // (F, I) of a stretch of tokens: its summed log forget gates, and what its input gates alone would
        // make of the maximum; stretches combine as (F1 + F2, max(I1 + F2, I2)).  Lanes beyond the chunk
        // hold the neutral stretch (0, -inf).
        float F = 0.f, I = -INFINITY;
        if (live) {
          I = cap * tanhf((grow[h] + par0) / cap);
          F = log_sigmoid_f32(cap * tanhf((grow[nh + h] + par1) / cap));
        }
        const float log_i = I, log_f = F;
#pragma unroll
        for (int off = 1; off < kWalkChunk; off <<= 1) {
          const float Fp = __shfl_up(F, off, kWave), Ip = __shfl_up(I, off, kWave);
          if (lane >= off) {
            I = fmaxf(Ip + F, I);
            F = Fp + F;
          }
        }
        const float m_t = fmaxf(m_run + F, I);
        float m_before = __shfl_up(m_t, 1, kWave);
        if (lane == 0) m_before = m_run;
        if (live) {
          a_s[lane] = expf(log_f + m_before - m_t);
          b_s[lane] = expf(log_i - m_t);
          e_s[lane] = expf(-m_t);
        }
        m_run = __shfl(m_t, nt - 1, kWave);
        if (PHASE == WALK_LOCAL) log_decay += __shfl(F, nt - 1, kWave);
      } else {
        float la = 0.f;
        if (live) {
          const float dt = softplus_f32(grow[h] + par0);
          la = par1 * dt;
          a_s[lane] = expf(la);
          b_s[lane] = dt;
        }
        if (PHASE == WALK_LOCAL) {
#pragma unroll
          for (int off = 1; off < kWalkChunk; off <<= 1) la += __shfl_xor(la, off, kWave);
          log_decay += la;
        }
      }
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float a = a_s[tt], b = b_s[tt];
      const float vj = v_s[tt][j];
      const float bv = b * vj;
      float acc = 0.f, nq = 0.f;
      const float4* k4 = reinterpret_cast<const float4*>(&k_s[tt][0]);
      const float4* q4 = reinterpret_cast<const float4*>(&q_s[PHASE == WALK_LOCAL ? 0 : tt][0]);
#pragma unroll
      for (int r4 = 0; r4 < RPL / 4; ++r4) {
        const float4 kk = k4[r4 * 8 + g], qq = q4[r4 * 8 + g];
        const float kr[4] = {kk.x, kk.y, kk.z, kk.w}, qr[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = r4 * 4 + i;
          S[r] = fmaf(kr[i], bv, a * S[r]);
          if (PHASE != WALK_LOCAL) acc = fmaf(S[r], qr[i], acc);
          if (MODE == WALK_EXP_GATES) {
            n[r] = fmaf(kr[i], b, a * n[r]);
            if (PHASE != WALK_LOCAL) nq = fmaf(n[r], qr[i], nq);
          }
        }
      }
      if (PHASE == WALK_LOCAL) continue;
      acc += __shfl_xor(acc, 8, kWave);
      acc += __shfl_xor(acc, 16, kWave);
      acc += __shfl_xor(acc, 32, kWave);
      float y;
      if (MODE == WALK_EXP_GATES) {
        nq += __shfl_xor(nq, 8, kWave);
        nq += __shfl_xor(nq, 16, kWave);
        nq += __shfl_xor(nq, 32, kWave);
        y = acc / (fmaxf(fabsf(nq), e_s[tt]) + kWalkFloor);
      } else if (MODE == WALK_FIXED_DECAY) {
        y = acc;
      } else {
        y = fmaf(par2, vj, acc);
      }
      if (g == 0 && c < dv) out[(size_t)(t0 + tt) * nh * dv + (size_t)h * dv + c] = y;
    }
  }
  if (PHASE == WALK_FINAL && !last) return;
  if (PHASE == WALK_LOCAL) {
    st = seg_local + seg_at;
    if (cb == 0 && lane == 0) seg_decay[(size_t)blockIdx.z * nh + h] = log_decay;
  }
#pragma unroll
  for (int r = 0; r < RPL; ++r) st[r * 64 + lane] = S[r];
  if (MODE == WALK_EXP_GATES) {
    if (j == 0) {
      float4* ndst = reinterpret_cast<float4*>(st + RPL * 64);
#pragma unroll
      for (int r4 = 0; r4 < RPL / 4; ++r4) ndst[r4 * 8 + g] = make_float4(n[r4 * 4], n[r4 * 4 + 1], n[r4 * 4 + 2], n[r4 * 4 + 3]);
    }
    if (lane == 0) st[RPL * 64 + DKP] = m_run;
  }
}

// The segments' start states, one entry's after the other: start(first) = the slot's state, start(s + 1) =
// what segment s makes of start(s).  A thread owns one float of a (head, 8 value columns) slice (of S or,
// for the gates, of n) and keeps it in a register; it asks for eight segments' local values before it
// uses the first (they do not depend on the chain), then moves along them.
constexpr int kCombineThreads = 256;
constexpr int kCombineAhead = 8;

template <int MODE>
__global__ __launch_bounds__(kCombineThreads) void state_walk_combine_kernel(
    const float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ ent_segs,
    const float* __restrict__ seg_local, float* __restrict__ seg_start, const float* __restrict__ seg_decay, int nh,
    int ncb, int dkp) {
  const int h = blockIdx.y, e = blockIdx.z;
  const int first = ent_segs[2 * e], count = ent_segs[2 * e + 1];
  if (count <= 0) return;
  const int slice = walk_slice_floats(dkp, MODE);
  const int moved = (dkp / 8) * 64 + (MODE == WALK_EXP_GATES ? dkp : 0);     // S and n; the maximum lies behind them
  const int idx = blockIdx.x * kCombineThreads + threadIdx.x;              // over the head's slices
  if (idx >= ncb * moved) return;
  const int cb = idx / moved, i = idx % moved;
  const size_t per_seg = (size_t)nh * ncb * slice;
  const size_t at = ((size_t)h * ncb + cb) * slice;
  const float* slot = state + (size_t)state_slots[e] * per_seg + at;
  float cur = slot[i];
  float m = MODE == WALK_EXP_GATES ? slot[moved] : 0.f;
  seg_start[(size_t)first * per_seg + at + i] = cur;
  if (MODE == WALK_EXP_GATES && i == 0) seg_start[(size_t)first * per_seg + at + moved] = m;
  for (int s0 = first; s0 + 1 < first + count; s0 += kCombineAhead) {
    const int n = min(kCombineAhead, first + count - 1 - s0);
    float loc[kCombineAhead], F[kCombineAhead], m_loc[kCombineAhead];
#pragma unroll
    for (int u = 0; u < kCombineAhead; ++u) {
      const int s = s0 + min(u, n - 1);                // (addresses clamped: no load behind a branch)
      loc[u] = seg_local[(size_t)s * per_seg + at + i];
      F[u] = seg_decay[(size_t)s * nh + h];
      m_loc[u] = MODE == WALK_EXP_GATES ? seg_local[(size_t)s * per_seg + at + moved] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kCombineAhead; ++u) {
      if (u < n) {
        float wa, wb = 1.f;
        if (MODE == WALK_EXP_GATES) {
          const float m_new = fmaxf(F[u] + m, m_loc[u]);
          wa = expf(F[u] + m - m_new);
          wb = expf(m_loc[u] - m_new);
          m = m_new;
        } else {
          wa = expf(F[u]);
        }
        cur = fmaf(wa, cur, wb * loc[u]);
        const size_t to = (size_t)(s0 + u + 1) * per_seg + at;
        seg_start[to + i] = cur;
        if (MODE == WALK_EXP_GATES && i == 0) seg_start[to + moved] = m;
      }
    }
  }
}

struct WalkArgs {
  const void* proj; int stride, q_off, k_off, v_off, heads_per_group;
  const float* gates; int gate_stride; const float *p0, *p1, *p2;
  float cap, q_scale; float* state; const int *state_slots, *cu_tokens; float* out;
  int n_entries, nh, dk, dv;
  const int *segs, *ent_segs; int n_segs; float *seg_local, *seg_start, *seg_decay;
  const int* positions; const float* inv_freq; int rot_dim; float k_scale;      // WALK_FIXED_DECAY
};

template <typename T, int RPL, int MODE, int PHASE>
static void launch_walk_phase(const WalkArgs& a, int ncb, int vec, hipStream_t stream) {
  dim3 grid(ncb, a.nh, PHASE == WALK_WHOLE ? a.n_entries : a.n_segs);
  state_walk_kernel<T, RPL, MODE, PHASE><<<grid, kWave, 0, stream>>>(
      (const T*)a.proj, a.stride, a.q_off, a.k_off, a.v_off, a.heads_per_group, a.gates, a.gate_stride, a.p0, a.p1, a.p2,
      a.cap, a.q_scale, a.state, a.state_slots, a.cu_tokens, a.out, a.nh, a.dk, a.dv, ncb, vec, a.segs, a.seg_local,
      a.seg_start, a.seg_decay, a.positions, a.inv_freq, a.rot_dim, a.k_scale);
}

template <typename T, int RPL, int MODE>
static int launch_walk_rpl(const WalkArgs& a, int ncb, int vec, hipStream_t stream) {
  if (!a.segs) {
    launch_walk_phase<T, RPL, MODE, WALK_WHOLE>(a, ncb, vec, stream);
    SHARPI_CHECK_LAUNCH();
    return SHARPI_OK;
  }
  launch_walk_phase<T, RPL, MODE, WALK_LOCAL>(a, ncb, vec, stream);
  SHARPI_CHECK_LAUNCH();
  const int moved = RPL * 64 + (MODE == WALK_EXP_GATES ? RPL * 8 : 0);
  state_walk_combine_kernel<MODE><<<dim3(ceil_div(ncb * moved, kCombineThreads), a.nh, a.n_entries), kCombineThreads, 0, stream>>>(
      a.state, a.state_slots, a.ent_segs, a.seg_local, a.seg_start, a.seg_decay, a.nh, ncb, RPL * 8);
  SHARPI_CHECK_LAUNCH();
  launch_walk_phase<T, RPL, MODE, WALK_FINAL>(a, ncb, vec, stream);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

template <typename T, int MODE>
static int launch_state_walk(const WalkArgs& a, hipStream_t stream) {
  const int ncb = ceil_div(a.dv, kWalkCols);
  constexpr int V = 16 / (int)sizeof(T);
  const int vec = a.dk % V == 0 && a.stride % V == 0 && a.q_off % V == 0 && a.k_off % V == 0 &&
                  reinterpret_cast<uintptr_t>(a.proj) % 16 == 0;
  if (a.dk <= 32) return launch_walk_rpl<T, 4, MODE>(a, ncb, vec, stream);
  if (a.dk <= 64) return launch_walk_rpl<T, 8, MODE>(a, ncb, vec, stream);
  if (a.dk <= 128) return launch_walk_rpl<T, 16, MODE>(a, ncb, vec, stream);
  if (a.dk <= 256) return launch_walk_rpl<T, 32, MODE>(a, ncb, vec, stream);
  return SHARPI_ERR_ARG;
}

static int state_walk_any(const WalkArgs& a, int dtype, int mode, hipStream_t stream) {
  if (a.n_entries <= 0) return SHARPI_OK;
  if (a.nh <= 0 || a.nh > 65535 || a.n_entries > 65535 || a.dk <= 0 || a.dk > 256 || a.dv <= 0 || a.heads_per_group <= 0) return SHARPI_ERR_ARG;
  if (mode != WALK_EXP_GATES && mode != WALK_STATE_SPACE && mode != WALK_FIXED_DECAY) return SHARPI_ERR_ARG;
  if (mode == WALK_FIXED_DECAY) {
    if (!a.p0 || a.rot_dim < 0 || (a.rot_dim & 1) || a.rot_dim > a.dk || (a.rot_dim > 0 && (!a.positions || !a.inv_freq))) return SHARPI_ERR_ARG;
  } else if (!a.gates || !a.p0 || !a.p1 || (mode == WALK_STATE_SPACE && !a.p2) || (mode == WALK_EXP_GATES && !(a.cap > 0.f))) {
    return SHARPI_ERR_ARG;
  }
  if (dtype != DT_F32 && dtype != DT_BF16) return SHARPI_ERR_ARG;
  if (a.segs && (!a.ent_segs || !a.seg_local || !a.seg_start || !a.seg_decay || a.n_segs < a.n_entries || a.n_segs > 65535)) return SHARPI_ERR_ARG;
  if (mode == WALK_EXP_GATES) {
    if (dtype == DT_F32) return launch_state_walk<float, WALK_EXP_GATES>(a, stream);
    return launch_state_walk<bf16_t, WALK_EXP_GATES>(a, stream);
  }
  if (mode == WALK_FIXED_DECAY) {
    if (dtype == DT_F32) return launch_state_walk<float, WALK_FIXED_DECAY>(a, stream);
    return launch_state_walk<bf16_t, WALK_FIXED_DECAY>(a, stream);
  }
  if (dtype == DT_F32) return launch_state_walk<float, WALK_STATE_SPACE>(a, stream);
  return launch_state_walk<bf16_t, WALK_STATE_SPACE>(a, stream);
}

// proj [T, stride] (dtype): q and k of head h at columns q_off / k_off + (h / heads_per_group) dk, v at
// v_off + h dv.  gates float [T, gate_stride]: WALK_EXP_GATES reads columns h (input gate) and nh + h
// (forget gate), p0 / p1 their biases [nh], cap the gates' cap; WALK_STATE_SPACE reads column h (the
// step size before its softplus), p0 its bias, p1 A_log, p2 D (all [nh]); WALK_FIXED_DECAY reads no gates:
// p0 the heads' decays [nh], k_scale the keys' scale, and positions int [T], inv_freq float [rot_dim / 2]
// turn the leading rot_dim elements of q and k (rot_dim 0: no rotation).  state float [slots, nh,
// ceil(dv / 8), slice]; out float [T, nh dv].
SHARPI_EXPORT int sharpi_state_walk(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off,
                                    int heads_per_group, const float* gates, int gate_stride, const float* p0,
                                    const float* p1, const float* p2, float cap, float q_scale, int mode, float* state,
                                    const int* state_slots, const int* cu_tokens, float* out, int n_entries, int nh,
                                    int dk, int dv, const int* positions, const float* inv_freq, int rot_dim, float k_scale,
                                    hipStream_t stream) {
  const WalkArgs a{proj, stride, q_off, k_off, v_off, heads_per_group, gates, gate_stride, p0, p1, p2, cap, q_scale, state,
                   state_slots, cu_tokens, out, n_entries, nh, dk, dv, nullptr, nullptr, 0, nullptr, nullptr, nullptr,
                   positions, inv_freq, rot_dim, k_scale};
  return state_walk_any(a, dtype, mode, stream);
}

// The same walk with long entries cut into segments that are walked side by side (results equal to
// rounding).  segs int [n_segs, 4] = (entry, first row, tokens, 1 if the entry's last), in the entries'
// order; ent_segs int [n_entries, 2] = (first segment, segments); seg_local and seg_start float [n_segs, nh,
// ceil(dv / 8), slice]; seg_decay float [n_segs, nh].
SHARPI_EXPORT int sharpi_state_walk_segmented(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off,
                                              int heads_per_group, const float* gates, int gate_stride, const float* p0,
                                              const float* p1, const float* p2, float cap, float q_scale, int mode,
                                              float* state, const int* state_slots, const int* cu_tokens, float* out,
                                              int n_entries, int nh, int dk, int dv, const int* segs, const int* ent_segs,
                                              int n_segs, float* seg_local, float* seg_start, float* seg_decay,
                                              const int* positions, const float* inv_freq, int rot_dim, float k_scale,
                                              hipStream_t stream) {
  if (!segs) return SHARPI_ERR_ARG;
  const WalkArgs a{proj, stride, q_off, k_off, v_off, heads_per_group, gates, gate_stride, p0, p1, p2, cap, q_scale, state,
                   state_slots, cu_tokens, out, n_entries, nh, dk, dv, segs, ent_segs, n_segs, seg_local, seg_start, seg_decay,
                   positions, inv_freq, rot_dim, k_scale};
  return state_walk_any(a, dtype, mode, stream);
}

// ---------------------------------------------------------------------------
// Behind a walk: o float [T, G * gd] in G equal parts, each divided by its root mean square, times a
// weight per channel, times a gate act(z) read from columns g_off.. of proj [T, stride] (act: 0 none,
// 1 SiLU, 2 sigmoid).  gate_first: the gate multiplies o BEFORE the statistics are taken (the norm
// then sees the gated values); otherwise after the weight.  A wave a (token, part).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float gate_value(int act, float z) {
  const float s = 1.0f / (1.0f + expf(-z));
  return act == 1 ? z * s : s;
}

template <typename T>
__global__ __launch_bounds__(256) void group_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                               float eps, const T* __restrict__ proj, int stride,
                                                               int g_off, int act, int gate_first, T* __restrict__ out,
                                                               int n_tokens, int G, int gd) {
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);     // (token, part), parts fastest
  const int lane = threadIdx.x & (kWave - 1);
  if (pair >= n_tokens * G) return;
  const int t = pair / G, p = pair % G;
  const float* x = o + (size_t)pair * gd;
  const T* gate = act ? proj + (size_t)t * stride + g_off + (size_t)p * gd : nullptr;
  float ss = 0.f;
  for (int d = lane; d < gd; d += kWave) {
    float v = x[d];
    if (gate && gate_first) v *= gate_value(act, to_f32<T>(gate[d]));
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)gd + eps);
  for (int d = lane; d < gd; d += kWave) {
    float v = x[d];
    if (gate && gate_first) v *= gate_value(act, to_f32<T>(gate[d]));
    float y = w ? v * inv * w[(size_t)p * gd + d] : v * inv;      // (w null: a norm without a weight)
    if (gate && !gate_first) y *= gate_value(act, to_f32<T>(gate[d]));
    out[(size_t)pair * gd + d] = from_f32<T>(y);
  }
}

SHARPI_EXPORT int sharpi_group_norm_gate(const float* o, const float* w, float eps, const void* proj, int dtype,
                                         int stride, int g_off, int act, int gate_first, void* out, int n_tokens, int G,
                                         int gd, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (G <= 0 || gd <= 0 || act < 0 || act > 2 || (act && !proj)) return SHARPI_ERR_ARG;
  const int blocks = ceil_div(n_tokens * G, 4);
  if (dtype == DT_F32)
    group_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>(o, w, eps, (const float*)proj, stride, g_off, act, gate_first,
                                                               (float*)out, n_tokens, G, gd);
  else if (dtype == DT_BF16)
    group_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, w, eps, (const bf16_t*)proj, stride, g_off, act,
                                                                gate_first, (bf16_t*)out, n_tokens, G, gd);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// A short causal convolution over time on C channels of proj [T, stride] (columns c_off..), with a
// bias, then SiLU: y_t = silu(b + sum_j w[:, j] u_(t - taps + 1 + j)) (w float [C, taps]; the last
// column is the current token's).  Before an entry's first row of the step the inputs come from the
// request's tail, float [slots, taps - 1, C] (its last taps - 1 inputs, oldest first; zeros for a new
// request).  A second kernel moves the tails on.  Sums in float, the current token's term last.
// ---------------------------------------------------------------------------
constexpr int kConvMaxTaps = 8;

template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(const T* __restrict__ proj, int stride, int c_off,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          int taps, const float* __restrict__ tail,
                                                          const int* __restrict__ state_slots,
                                                          const int* __restrict__ entry_of_token,
                                                          const int* __restrict__ cu_tokens, T* __restrict__ out, int C) {
  const int t = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= C) return;
  const int e = entry_of_token[t];
  const int local = t - cu_tokens[e];
  const float* tl = tail ? tail + (size_t)state_slots[e] * (taps - 1) * C : nullptr;
  float acc = bias ? bias[ch] : 0.f;
  for (int jx = 0; jx < taps; ++jx) {
    const int back = taps - 1 - jx;           // how many tokens before this one
    float u;
    if (back <= local) u = to_f32<T>(proj[(size_t)(t - back) * stride + c_off + ch]);
    else u = tl[(size_t)(taps - 1 + local - back) * C + ch];
    acc = fmaf(w[(size_t)ch * taps + jx], u, acc);
  }
  out[(size_t)t * C + ch] = from_f32<T>(acc / (1.0f + expf(-acc)));
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_tail_kernel(const T* __restrict__ proj, int stride, int c_off, int taps,
                                                               float* __restrict__ tail, const int* __restrict__ state_slots,
                                                               const int* __restrict__ cu_tokens, int C) {
  const int e = blockIdx.x;
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= C) return;
  const int first = cu_tokens[e], L = cu_tokens[e + 1] - first;
  if (L <= 0) return;
  float* tl = tail + (size_t)state_slots[e] * (taps - 1) * C;
  float keep[kConvMaxTaps];
  for (int i = 0; i < taps - 1; ++i) {        // the new row i is the input at local index L - (taps - 1) + i
    const int li = L - (taps - 1) + i;
    keep[i] = li >= 0 ? to_f32<T>(proj[(size_t)(first + li) * stride + c_off + ch]) : tl[(size_t)(taps - 1 + li) * C + ch];
  }
  for (int i = 0; i < taps - 1; ++i) tl[(size_t)i * C + ch] = keep[i];
}

SHARPI_EXPORT int sharpi_short_conv(const void* proj, int dtype, int stride, int c_off, const float* w, const float* bias,
                                    int taps, float* tail, const int* state_slots, const int* entry_of_token,
                                    const int* cu_tokens, void* out, int n_tokens, int n_entries, int C, int update_tail,
                                    hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (C <= 0 || taps < 1 || taps > kConvMaxTaps || (taps > 1 && !tail) || n_entries <= 0 || ceil_div(C, 256) > 65535) return SHARPI_ERR_ARG;
  if (dtype != DT_F32 && dtype != DT_BF16) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens, ceil_div(C, 256)), tgrid(n_entries, ceil_div(C, 256));
  if (dtype == DT_F32) {
    short_conv_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, stride, c_off, w, bias, taps, tail, state_slots,
                                                        entry_of_token, cu_tokens, (float*)out, C);
    SHARPI_CHECK_LAUNCH();
    if (taps > 1 && update_tail)
      short_conv_tail_kernel<float><<<tgrid, 256, 0, stream>>>((const float*)proj, stride, c_off, taps, tail, state_slots,
                                                                cu_tokens, C);
  } else {
    short_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)proj, stride, c_off, w, bias, taps, tail,
                                                         state_slots, entry_of_token, cu_tokens, (bf16_t*)out, C);
    SHARPI_CHECK_LAUNCH();
    if (taps > 1 && update_tail)
      short_conv_tail_kernel<bf16_t><<<tgrid, 256, 0, stream>>>((const bf16_t*)proj, stride, c_off, taps, tail, state_slots,
                                                                 cu_tokens, C);
  }
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
