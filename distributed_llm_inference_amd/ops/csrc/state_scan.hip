// Linear recurrences over a per-sequence matrix state, token by token, everything in fp32. One kernel, two rules:
//
//   rule 0, generalised delta rule, state S [d, d] per head:
//       u = k / sqrt(sum k^2 + 1e-6);  S <- diag(w) S - (a u) (u^T S) + k v^T  (S on the right is the state before the token);  o = S^T r
//       w = exp(-exp(-1/2) sigmoid(wz + w0)),  a = sigmoid(za + ba)   (a decay and a removal rate per key channel)
//   rule 1, matrix memory with exponential gates, state S [d, dv], normaliser n [d], running maximum m per head:
//       i = cap tanh((zi + bi) / cap),  f = logsigmoid(cap tanh((zf + bf) / cap)),  m' = max(f + m, i)
//       S <- exp(f + m - m') S + exp(i - m') k v^T,  n the same with k alone;  the kernel writes the raw read-out S^T q,
//       n . q and exp(-m') per head ([dv | n.q | exp(-m')] per head in `o`); the division by max(|n . q|, exp(-m')) + 1e-6
//       happens where the read-out is normalised per head. n is kept as one more column of the state (its "value" is 1).
//
// Both rules act on every column of the state alone, so the work is split by columns: a workgroup owns (sequence, head,
// a block of CB columns), a column's d rows live in the registers of R neighbouring lanes (16 rows each, rows beyond d are
// zero), the dot products over d are finished with R-lane shuffles. The step's tokens go through LDS in chunks: all threads
// load a chunk's per-token vectors and evaluate the gates (a token per 16 lanes), then every lane walks the chunk's tokens
// over its registers. A step is ragged: sequence b brings q_start[b+1] - q_start[b] tokens after ctx[b] earlier ones and
// owns state slot slots[b]; ctx 0 starts from zeros (m from 0) whatever the slot held, so slots change hands without clearing.
// The running maximum is kept in kScanMaxBlocks copies per (slot, head): the workgroup of column block zb (of ZB) reads copy zb
// and writes every copy whose index is zb modulo ZB, so that no workgroup reads what another one of the same launch writes,
// and a later step that splits the columns into another number of blocks still finds every copy it reads up to date.
#include <stdlib.h>
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kScanRows = 16;            // state rows per lane
constexpr int kScanMaxBlocks = 128;      // copies of the running maximum per (slot, head)

struct ScanArgs {
  float* o; long ldo;
  const float* z; long ldz;
  const float* wz; long ldw;
  float* state; float* mstate;
  const float* b0; const float* b1;
  const int* q_start; const int* ctx; const int* slots;
  int H, d, dv, NC, R, CB, CH, DP, state_rows, ZB;
  int col_q, col_k, col_v, col_a, col_i, col_f;
  float cap, qscale;
  int vec4;       // every row and column offset of z / wz is a multiple of 4 floats and 16-byte aligned: 16-byte loads
  int quick;      // gates through the hardware's exp2 / reciprocal (about 1 ulp) instead of the library functions
};

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float logsigmoidf_(float x) { return x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x)); }
// the same gates on the hardware's transcendental instructions: still fp32, about 1 ulp each; the library versions are
// a few dozen instructions per value, which is most of what a chunk costs besides walking its tokens
__device__ __forceinline__ float q_exp(float x) { return __expf(x); }
__device__ __forceinline__ float q_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
__device__ __forceinline__ float q_tanh(float x) { return 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f); }

template <int RULE>
__global__ __launch_bounds__(256) void state_scan_kernel(ScanArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int NV = RULE == 0 ? 5 : 2;
  const int b = blockIdx.x, h = blockIdx.y, zb = blockIdx.z;
  const int t0 = p.q_start[b], n = p.q_start[b + 1] - t0, c0 = p.ctx[b], slot = p.slots[b];
  if (n <= 0 || slot < 0 || slot >= p.state_rows) return;
  const int tid = threadIdx.x, R = p.R, CB = p.CB, DP = p.DP, d = p.d, NC = p.NC;
  const int c = tid / R, rg = tid % R, j = zb * CB + c;
  const bool col_ok = j < NC;
  float* vec = lds;                                  // [CH][NV][DP]
  float* vals = vec + (long)p.CH * NV * DP;          // [CH][CB]
  float* sc = vals + (long)p.CH * CB;                // [CH][4]: rule 1: log i, log f -> keep, put, exp(-m')
  float* S = p.state + ((long)slot * p.H + h) * (long)d * NC;
  float s[kScanRows];
#pragma unroll
  for (int e = 0; e < kScanRows; ++e) {
    const int row = rg * kScanRows + e;
    s[e] = (c0 > 0 && col_ok && row < d) ? S[(long)row * NC + j] : 0.f;
  }
  float* mp = p.mstate ? p.mstate + ((long)slot * p.H + h) * kScanMaxBlocks + zb : nullptr;
  float m_run = (RULE == 1 && c0 > 0) ? mp[0] : 0.f;         // (only thread 0's copy is used)
  const int tt = tid >> 4, sub = tid & 15;
  const int hd = h * d;
  for (int ch0 = 0; ch0 < n; ch0 += p.CH) {
    const int nt = min(p.CH, n - ch0);
    __syncthreads();                                 // the previous chunk has been consumed
    if (tt < nt) {
      const long t = t0 + ch0 + tt;
      const float* zr = p.z + t * p.ldz;
      float* v0 = vec + (long)tt * NV * DP;
      if constexpr (RULE == 0) {
        const float* wr = p.wz + t * p.ldw;
        float ksq = 0.f;
        for (int i = sub; i < DP; i += 16) {
          float k = 0.f, r = 0.f, a = 0.f, w = 0.f;
          if (i < d) {
            k = zr[p.col_k + hd + i]; r = zr[p.col_q + hd + i];
            a = sigmoidf_(zr[p.col_a + hd + i] + p.b0[hd + i]);
            w = expf(-0.6065306597126334f * sigmoidf_(wr[hd + i] + p.b1[hd + i]));
          }
          ksq += k * k;
          v0[i] = w; v0[DP + i] = a; v0[3 * DP + i] = k; v0[4 * DP + i] = r;
        }
#pragma unroll
        for (int o = 8; o >= 1; o >>= 1) ksq += __shfl_xor(ksq, o, 64);
        const float inv = rsqrtf(ksq + 1e-6f);
        for (int i = sub; i < DP; i += 16) {          // (each lane re-reads what it wrote itself)
          const float u = v0[3 * DP + i] * inv;
          v0[DP + i] *= u; v0[2 * DP + i] = u;
        }
      } else {
        for (int i = sub; i < DP; i += 16) {
          v0[i] = i < d ? zr[p.col_k + hd + i] : 0.f;
          v0[DP + i] = i < d ? zr[p.col_q + hd + i] * p.qscale : 0.f;
        }
        if (sub == 0) {
          sc[tt * 4] = p.cap * tanhf((zr[p.col_i + h] + p.b0[h]) / p.cap);
          sc[tt * 4 + 1] = logsigmoidf_(p.cap * tanhf((zr[p.col_f + h] + p.b0[p.H + h]) / p.cap));
        }
      }
      for (int cc = sub; cc < CB; cc += 16) {
        const int jj = zb * CB + cc;
        float v = 0.f;
        if (jj < p.dv) v = zr[p.col_v + h * p.dv + jj];
        else if (RULE == 1 && jj == p.dv) v = 1.f;
        vals[tt * CB + cc] = v;
      }
    }
    if constexpr (RULE == 1) {
      __syncthreads();
      if (tid == 0)
        for (int q = 0; q < nt; ++q) {
          const float li = sc[q * 4], lf = sc[q * 4 + 1];
          const float m_new = fmaxf(lf + m_run, li);
          sc[q * 4] = expf(lf + m_run - m_new); sc[q * 4 + 1] = expf(li - m_new); sc[q * 4 + 2] = expf(-m_new);
          m_run = m_new;
        }
    }
    __syncthreads();
    for (int q = 0; q < nt; ++q) {
      const float* v0 = vec + (long)q * NV * DP + rg * kScanRows;
      const float v = vals[q * CB + c];
      float out = 0.f;
      if constexpr (RULE == 0) {
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < kScanRows; ++e) dot += v0[2 * DP + e] * s[e];
        for (int o = 1; o < R; o <<= 1) dot += __shfl_xor(dot, o, 64);
#pragma unroll
        for (int e = 0; e < kScanRows; ++e) {
          s[e] = v0[e] * s[e] - v0[DP + e] * dot + v0[3 * DP + e] * v;
          out += v0[4 * DP + e] * s[e];
        }
      } else {
        const float keep = sc[q * 4], put = sc[q * 4 + 1] * v;
#pragma unroll
        for (int e = 0; e < kScanRows; ++e) {
          s[e] = keep * s[e] + put * v0[e];
          out += v0[DP + e] * s[e];
        }
      }
      for (int o = 1; o < R; o <<= 1) out += __shfl_xor(out, o, 64);
      if (rg == 0 && col_ok) {
        float* orow = p.o + (long)(t0 + ch0 + q) * p.ldo;
        if constexpr (RULE == 0) orow[h * p.dv + j] = out;
        else {
          orow[h * (p.dv + 2) + j] = out;
          if (j == p.dv) orow[h * (p.dv + 2) + p.dv + 1] = sc[q * 4 + 2];
        }
      }
    }
  }
  if (col_ok) {
#pragma unroll
    for (int e = 0; e < kScanRows; ++e) {
      const int row = rg * kScanRows + e;
      if (row < d) S[(long)row * NC + j] = s[e];
    }
  }
  if (RULE == 1 && tid == 0)
    for (int i = zb; i < kScanMaxBlocks; i += p.ZB) mp[i - zb] = m_run;
}

// The same walk for key sizes up to 128 with everything that sits on the chain from one token to the next made short. A
// workgroup's four waves each sit alone on a SIMD, so nothing hides latency: the time per token IS the dependent chain. Here
// a column's rows are spread over R <= 16 lanes known at compile time (16 rows each, or 8 when a step has so few sequences
// that narrower column blocks are what fills the chip; in LDS every lane's rows are followed by 4 words
// of padding, so that the 16-byte reads of lanes with different rows fall into different banks: without it the reads of a wave
// collide four ways and the LDS pipe, not the arithmetic, sets the time per token), the two sums over the rows run as four
// independent chains and finish with data-parallel-primitive moves between neighbouring lanes (no LDS round trip), the NEXT
// chunk's inputs are fetched into registers before the current chunk is walked and become LDS contents (gates evaluated, key
// normalised) after it. Rule 1's running maximum is a prefix scan over the chunk's tokens in the (max, +) algebra —
// m -> max(a + m, b) composes as (a1 + a2, max(a2 + b1, b2)) — done by the first 16 lanes of every wave with shuffles, so it
// costs no barrier and no serial loop; the per-token factors then travel by lane broadcast.
constexpr int kFastPad = 4;

template <int RULE, int R, int kFastRows>
__global__ __launch_bounds__(256) void state_scan_fast_kernel(ScanArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int NV = RULE == 0 ? 5 : 2, CB = 256 / R, DP = (kFastRows + kFastPad) * R, CH = 16, VPL = CB / 16, EL = kFastRows * R / 16;
  auto at = [](int row) { return row + (row / kFastRows) * kFastPad; };      // a row's place in a padded vector
  const int b = blockIdx.x, h = blockIdx.y, zb = blockIdx.z;
  const int t0 = p.q_start[b], n = p.q_start[b + 1] - t0, c0 = p.ctx[b], slot = p.slots[b];
  if (n <= 0 || slot < 0 || slot >= p.state_rows) return;
  const int tid = threadIdx.x, d = p.d, NC = p.NC;
  const int c = tid / R, rg = tid % R, j = zb * CB + c;
  const bool col_ok = j < NC;
  float* vec = lds;                                  // [CH][NV][DP]
  float* vals = vec + CH * NV * DP;                  // [CH][CB]
  float* sc = vals + CH * CB;                        // [CH][2]: rule 1: log i, log f
  float* obuf = sc + CH * 2;                         // [CH][CB + 1]: the chunk's read-outs (and exp(-m')) until they are stored
  float* S = p.state + ((long)slot * p.H + h) * (long)d * NC;
  float s[kFastRows];
#pragma unroll
  for (int e = 0; e < kFastRows; ++e) {
    const int row = rg * kFastRows + e;
    s[e] = (c0 > 0 && col_ok && row < d) ? S[(long)row * NC + j] : 0.f;
  }
  float* mp = p.mstate ? p.mstate + ((long)slot * p.H + h) * kScanMaxBlocks + zb : nullptr;
  float m_run = 0.f;
  if constexpr (RULE == 1) m_run = c0 > 0 ? mp[0] : 0.f;
  const int tt = tid >> 4, sub = tid & 15, hd = h * d, lane = tid & 63;
  // Inputs on their way from memory: D chunks ahead, a register set each. All memory traffic of a chunk is issued at ONE
  // point, between the two barriers: the read-outs of the chunk just walked (they wait in LDS) and the fetch of the chunk
  // after the next. The vector-memory counter is a single in-order count, and a wait for fetched inputs behind a loop of
  // conditional stores is a wait for everything; issued together and a whole walk ahead of the next wait, nothing stalls.
  constexpr int D = 1;
  struct Pre { float pa[EL], pb[EL], pc[RULE == 0 ? EL : 1], pd[RULE == 0 ? EL : 1], pv[VPL], pi, pf; };
  Pre pre[D];

  // the biases of this lane's rows are the same for every token: read once
  [[maybe_unused]] float ba[RULE == 0 ? EL : 1], bw[RULE == 0 ? EL : 1];
  if constexpr (RULE == 0) {
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const int i = sub * EL + e;
      ba[e] = i < d ? p.b0[hd + i] : 0.f;
      bw[e] = i < d ? p.b1[hd + i] : 0.f;
    }
  }
  // (a chunk's inputs are a few kilobytes per workgroup; fetched one float per lane and instruction they are dozens of
  // poorly coalesced requests per wave and the fetch, not the walk, sets the time per chunk: 16 bytes per lane where the
  // layout allows)
  auto row4 = [&](float (&dst)[EL], const float* src) {
    if constexpr (EL % 4 == 0) {
      if (p.vec4) {
#pragma unroll
        for (int e = 0; e < EL; e += 4) {
          const int i = sub * EL + e;
          const f32x4 t = i < d ? *reinterpret_cast<const f32x4*>(src + i) : f32x4{0.f, 0.f, 0.f, 0.f};
          dst[e] = t.x; dst[e + 1] = t.y; dst[e + 2] = t.z; dst[e + 3] = t.w;
        }
        return;
      }
    }
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const int i = sub * EL + e;
      dst[e] = i < d ? src[i] : 0.f;
    }
  };
  auto prefetch = [&](Pre& r, int ch0) {
    if (tt >= min(CH, n - ch0)) return;
    const long t = t0 + ch0 + tt;
    const float* zr = p.z + t * p.ldz;
    row4(r.pa, zr + p.col_k + hd);
    row4(r.pb, zr + p.col_q + hd);
    if constexpr (RULE == 0) {
      row4(r.pc, zr + p.col_a + hd);
      row4(r.pd, p.wz + t * p.ldw + hd);
#pragma unroll
      for (int e = 0; e < EL; ++e) { r.pc[e] += ba[e]; r.pd[e] += bw[e]; }
    }
#pragma unroll
    for (int e = 0; e < VPL; ++e) {
      const int jj = zb * CB + sub * VPL + e;
      r.pv[e] = jj < p.dv ? zr[p.col_v + h * p.dv + jj] : ((RULE == 1 && jj == p.dv) ? 1.f : 0.f);
    }
    if constexpr (RULE == 1) {
      if (sub == 0) { r.pi = zr[p.col_i + h] + p.b0[h]; r.pf = zr[p.col_f + h] + p.b0[p.H + h]; }
    }
  };
  auto commit = [&](const Pre& r, int nt) {
    if (tt >= nt) return;
    const float (&pa)[EL] = r.pa; const float (&pb)[EL] = r.pb; const auto& pc = r.pc; const auto& pd = r.pd; const float (&pv)[VPL] = r.pv;
    const float pi = r.pi, pf = r.pf;
    float* vt = vec + tt * NV * DP;
    if constexpr (RULE == 0) {
      float ksq = 0.f;
#pragma unroll
      for (int e = 0; e < EL; ++e) ksq += pa[e] * pa[e];
      ksq = group_sum<16>(ksq);
      const float inv = rsqrtf(ksq + 1e-6f);
#pragma unroll
      for (int e = 0; e < EL; ++e) {
        const bool ok = sub * EL + e < d;
        const float u = pa[e] * inv;
        float* v0 = vt + at(sub * EL + e);
        const float wv = p.quick ? q_exp(-0.6065306597126334f * q_sigmoid(pd[e])) : expf(-0.6065306597126334f * sigmoidf_(pd[e]));
        const float av = p.quick ? q_sigmoid(pc[e]) : sigmoidf_(pc[e]);
        v0[0] = ok ? wv : 0.f;
        v0[DP] = ok ? av * u : 0.f;
        v0[2 * DP] = u; v0[3 * DP] = pa[e]; v0[4 * DP] = pb[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < EL; ++e) { float* v0 = vt + at(sub * EL + e); v0[0] = pa[e]; v0[DP] = pb[e] * p.qscale; }
      if (sub == 0) {
        sc[tt * 2] = p.cap * (p.quick ? q_tanh(pi / p.cap) : tanhf(pi / p.cap));
        sc[tt * 2 + 1] = logsigmoidf_(p.cap * (p.quick ? q_tanh(pf / p.cap) : tanhf(pf / p.cap)));
      }
    }
#pragma unroll
    for (int e = 0; e < VPL; ++e) vals[tt * CB + sub * VPL + e] = pv[e];
  };

  auto flush = [&](int ch0, int nt) {                // the read-outs of the chunk that starts at ch0, from LDS to memory
    constexpr int HS = RULE == 0 ? 0 : 2;
    for (int i = tid; i < nt * CB; i += 256) {
      const int q = i / CB, cc = i % CB, jj = zb * CB + cc;
      if (jj < NC) p.o[(long)(t0 + ch0 + q) * p.ldo + h * (p.dv + HS) + jj] = obuf[q * (CB + 1) + cc];
    }
    if constexpr (RULE == 1) {
      if (tid < nt && zb * CB <= p.dv && p.dv < (zb + 1) * CB)
        p.o[(long)(t0 + ch0 + tid) * p.ldo + h * (p.dv + 2) + p.dv + 1] = obuf[tid * (CB + 1) + CB];
    }
  };
  auto chunk = [&](Pre& pr, int ch0) {
    const int nt = min(CH, n - ch0);
    __syncthreads();                                 // the previous chunk has been walked
    commit(pr, nt);
    if (ch0 > 0) flush(ch0 - CH, CH);
    if (ch0 + D * CH < n) prefetch(pr, ch0 + D * CH);      // in flight while this chunk is walked
    __syncthreads();
    [[maybe_unused]] float keepv = 1.f, putv = 0.f, emv = 1.f;
    if constexpr (RULE == 1) {
      const bool live = lane < nt;
      const float lf = live ? sc[(lane & 15) * 2 + 1] : 0.f, li = live ? sc[(lane & 15) * 2] : -INFINITY;
      float a = lf, bb = li;                         // the token's own map m -> max(a + m, b); lanes past the chunk: the identity
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) {
        const float ea = __shfl_up(a, o, 64), eb = __shfl_up(bb, o, 64);
        if ((lane & 15) >= o) { bb = fmaxf(a + eb, bb); a = ea + a; }
      }
      const float m_t = fmaxf(a + m_run, bb);
      float m_prev = __shfl_up(m_t, 1, 64);
      if ((lane & 15) == 0) m_prev = m_run;
      if (p.quick) { keepv = q_exp(lf + m_prev - m_t); putv = q_exp(li - m_t); emv = q_exp(-m_t); }
      else { keepv = expf(lf + m_prev - m_t); putv = expf(li - m_t); emv = expf(-m_t); }
      m_run = __shfl(m_t, nt - 1, 64);
    }
    // two register sets: the vectors of token q + 1 are read from LDS while token q is applied
    float va[NV][kFastRows], vb[NV][kFastRows], xa, xb = 0.f;
    auto fetch = [&](float (&dst)[NV][kFastRows], float& x, int q) {
      const float* v0 = vec + q * NV * DP + rg * (kFastRows + kFastPad);
#pragma unroll
      for (int k = 0; k < NV; ++k)
#pragma unroll
        for (int e = 0; e < kFastRows; e += 4) {
          const f32x4 t = *reinterpret_cast<const f32x4*>(v0 + k * DP + e);
          dst[k][e] = t.x; dst[k][e + 1] = t.y; dst[k][e + 2] = t.z; dst[k][e + 3] = t.w;
        }
      x = vals[q * CB + c];
    };
    auto apply = [&](const float (&w)[NV][kFastRows], float v, int q) {
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (RULE == 0) {
        float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < kFastRows; ++e) d4[e & 3] += w[2][e] * s[e];
        const float dot = group_sum<R>((d4[0] + d4[1]) + (d4[2] + d4[3]));
#pragma unroll
        for (int e = 0; e < kFastRows; ++e) {
          s[e] = w[0][e] * s[e] - w[1][e] * dot + w[3][e] * v;
          o4[e & 3] += w[4][e] * s[e];
        }
      } else {
        const float keep = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, keepv), q));
        const float put = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, putv), q)) * v;
#pragma unroll
        for (int e = 0; e < kFastRows; ++e) {
          s[e] = keep * s[e] + put * w[0][e];
          o4[e & 3] += w[1][e] * s[e];
        }
      }
      const float out = group_sum<R>((o4[0] + o4[1]) + (o4[2] + o4[3]));
      if (rg == 0) {
        obuf[q * (CB + 1) + c] = out;
        if constexpr (RULE == 1) {
          if (j == p.dv) obuf[q * (CB + 1) + CB] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, emv), q));
        }
      }
    };
    fetch(va, xa, 0);
    for (int q = 0; q < nt; q += 2) {
      if (q + 1 < nt) fetch(vb, xb, q + 1);
      apply(va, xa, q);
      if (q + 1 < nt) {
        if (q + 2 < nt) fetch(va, xa, q + 2);
        apply(vb, xb, q + 1);
      }
    }
  };
#pragma unroll
  for (int i = 0; i < D; ++i)
    if (i * CH < n) prefetch(pre[i], i * CH);
  for (int base = 0; base < n; base += D * CH) {
#pragma unroll
    for (int i = 0; i < D; ++i)
      if (base + i * CH < n) chunk(pre[i], base + i * CH);
  }
  __syncthreads();
  flush((n - 1) / CH * CH, n - (n - 1) / CH * CH);
  if (col_ok) {
#pragma unroll
    for (int e = 0; e < kFastRows; ++e) {
      const int row = rg * kFastRows + e;
      if (row < d) S[(long)row * NC + j] = s[e];
    }
  }
  if constexpr (RULE == 1) {
    if (tid == 0)
      for (int i = zb; i < kScanMaxBlocks; i += p.ZB) mp[i - zb] = m_run;
  }
}

template <int RULE, int ROWS>
static void launch_scan_fast(const ScanArgs& p, int R, dim3 grid, hipStream_t stream) {
  const int nv = RULE == 0 ? 5 : 2;
  const size_t lds = (size_t)16 * (nv * (ROWS + kFastPad) * R + 2 * (256 / R) + 3) * sizeof(float);
  if constexpr (ROWS == 16) {
    if (R == 1) { hipLaunchKernelGGL((state_scan_fast_kernel<RULE, 1, 16>), grid, dim3(256), lds, stream, p); return; }
  } else {
    if (R == 16) { hipLaunchKernelGGL((state_scan_fast_kernel<RULE, 16, 8>), grid, dim3(256), lds, stream, p); return; }
  }
  if (R == 2) hipLaunchKernelGGL((state_scan_fast_kernel<RULE, 2, ROWS>), grid, dim3(256), lds, stream, p);
  else if (R == 4) hipLaunchKernelGGL((state_scan_fast_kernel<RULE, 4, ROWS>), grid, dim3(256), lds, stream, p);
  else hipLaunchKernelGGL((state_scan_fast_kernel<RULE, 8, ROWS>), grid, dim3(256), lds, stream, p);
}

}  // namespace dlia

// Column blocks a (d, columns) state is split into: the launch shape depends on the sizes only, never on the step.
extern "C" int dlia_state_scan_blocks(int d, int ncols) {
  int R = 1;
  while (R * dlia::kScanRows < d) R <<= 1;
  if (R > 64) return -1;
  const int CB = 256 / R;
  return (ncols + CB - 1) / CB;
}

extern "C" int dlia_state_scan(int rule, float* o, long ldo, const float* z, long ldz, const float* wz, long ldw, float* state,
                               float* mstate, const float* b0, const float* b1, const int* q_start, const int* ctx,
                               const int* slots, int B, int H, int d, int dv, int state_rows, int col_q, int col_k, int col_v,
                               int col_a, int col_i, int col_f, float cap, float qscale, int max_q, int quick, hipStream_t stream) {
  if (B <= 0) return 0;
  dlia::ScanArgs p;
  p.o = o; p.ldo = ldo; p.z = z; p.ldz = ldz; p.wz = wz; p.ldw = ldw; p.state = state; p.mstate = mstate; p.b0 = b0; p.b1 = b1;
  p.q_start = q_start; p.ctx = ctx; p.slots = slots; p.H = H; p.d = d; p.dv = dv; p.NC = rule == 0 ? dv : dv + 1;
  int R = 1;
  while (R * dlia::kScanRows < d) R <<= 1;
  if (R > 64) return 1;
  p.R = R; p.CB = 256 / R; p.DP = R * dlia::kScanRows; p.state_rows = state_rows;
  const int nv = rule == 0 ? 5 : 2;
  const int per_token = nv * p.DP + p.CB + 4;
  int CH = 12000 / per_token;
  p.CH = CH > 16 ? 16 : (CH < 1 ? 1 : CH);
  p.col_q = col_q; p.col_k = col_k; p.col_v = col_v; p.col_a = col_a; p.col_i = col_i; p.col_f = col_f; p.cap = cap; p.qscale = qscale; p.quick = quick;
  {
    auto al = [](const void* q) { return (uintptr_t)q % 16 == 0; };
    const bool cols = col_q % 4 == 0 && col_k % 4 == 0 && (rule != 0 || col_a % 4 == 0) && d % 4 == 0;
    p.vec4 = cols && ldz % 4 == 0 && al(z) && (rule != 0 || (ldw % 4 == 0 && al(wz)));
  }
  const int ZB = (p.NC + p.CB - 1) / p.CB;
  if (ZB > dlia::kScanMaxBlocks / 2) return 2;
  p.ZB = ZB;
  const size_t lds = (size_t)p.CH * per_token * sizeof(float);
  const dim3 grid(B, H, ZB);
  static const bool fast_on = [] { const char* e = getenv("DLIA_SCAN_FAST"); return !(e && atoi(e) == 0); }();
  // (steps of few tokens per sequence — decoding — run many workgroups at once: there the kernel that needs a third of the
  // registers keeps more of them resident, and there is no chain of tokens to shorten)
  if (d <= 128 && fast_on && max_q >= 8) {
    // few workgroups (one long prompt): 8 rows per lane, twice the column blocks, half the work per token and lane
    const bool narrow = d > 8 && (long)B * H * ZB < 192;
    const int rows = narrow ? 8 : 16;
    int Rf = narrow ? 2 : 1;
    while (Rf * rows < d) Rf <<= 1;
    p.ZB = (p.NC + 256 / Rf - 1) / (256 / Rf);
    const dim3 gridf(B, H, p.ZB);
    if (narrow) { if (rule == 0) dlia::launch_scan_fast<0, 8>(p, Rf, gridf, stream); else dlia::launch_scan_fast<1, 8>(p, Rf, gridf, stream); }
    else { if (rule == 0) dlia::launch_scan_fast<0, 16>(p, Rf, gridf, stream); else dlia::launch_scan_fast<1, 16>(p, Rf, gridf, stream); }
    return 0;
  }
  if (rule == 0)
    hipLaunchKernelGGL(dlia::state_scan_kernel<0>, grid, dim3(256), lds, stream, p);
  else
    hipLaunchKernelGGL(dlia::state_scan_kernel<1>, grid, dim3(256), lds, stream, p);
  return 0;
}
