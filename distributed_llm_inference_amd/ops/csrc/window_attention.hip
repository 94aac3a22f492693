// Paged attention for mixers whose sizes and mask are free parameters: queries / keys of `d`, values of `dv`
// (any sizes), an optional sliding window (a query at position i sees the keys j with 0 <= i - j < window), an
// optional softmax sink (one more term exp(0), or exp of a learned number per head, in the denominator, with no value),
// no rotation, the score scale given. Optional per head: a learned factor on the scaled scores, a bias per distance i - j
// (a table [distances, heads], added after scale and factor), a sigmoid gate on the head's output (one logit per token, head). Scores, the softmax and the weighted sum are fp32; the cache holds the compute type (bf16 or fp32).
//
// Cache layout per layer: K [block][kv head][32][d], V [block][kv head][32][dv], plain rows, blocks of 32 tokens
// addressed through the stage's block table (the same table and block ids as every other layer's cache).
//
// kv_store: one workgroup per new token. Reads the fp32 output of the fused q|k|v projection, blends the values
// with those of the stack's first value-mixing layer (mix 1: this IS that layer, remember v; mix 2:
// v <- (1 - lam) v + lam v_first) and writes k and the blended v into the token's cache row.
//
// window_attention: one wave per (new token, query head). Lanes split the keys of a 64-key step for the scores
// (each lane one dot product over d against q held in LDS), then split the value columns for the weighted sum,
// the weights travelling by lane shuffle. Online softmax across steps; the sink starts it at m = 0, l = 1.
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kWinBlock = 32;       // tokens per cache block (the stage's KV_BLOCK)
constexpr int kWinMaxD = 512;       // largest d / dv

template <typename T>
__global__ __launch_bounds__(256) void kv_store_kernel(
    const float* __restrict__ qkv, float* __restrict__ vfirst, const float* __restrict__ lam_p, int mix,
    T* __restrict__ kcache, T* __restrict__ vcache, const int* __restrict__ tok_pos, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, int num_blocks, int table_rows, int G, int d, int dv, int q_cols,
    long ld) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t], slot = tok_seq[t];
  const float* row = qkv + (long)t * ld + q_cols;
  const int kn = G * d, vn = G * dv;
  const float lam = mix == 2 ? lam_p[0] : 0.f;
  int blk = -1;
  if (slot >= 0 && slot < table_rows && pos >= 0 && pos / kWinBlock < max_blocks) blk = block_table[(long)slot * max_blocks + pos / kWinBlock];
  const bool store = blk >= 0 && blk < num_blocks;
  const int off = pos % kWinBlock;
  if (store)
    for (int i = threadIdx.x; i < kn; i += 256) {
      const int g = i / d, c = i % d;
      kcache[(((long)blk * G + g) * kWinBlock + off) * d + c] = (T)row[i];
    }
  for (int i = threadIdx.x; i < vn; i += 256) {
    float v = row[kn + i];
    if (mix == 1) vfirst[(long)t * vn + i] = v;
    if (mix == 2) v = (1.f - lam) * v + lam * vfirst[(long)t * vn + i];
    if (store) {
      const int g = i / dv, c = i % dv;
      vcache[(((long)blk * G + g) * kWinBlock + off) * dv + c] = (T)v;
    }
  }
}

template <typename T, typename OT>
__global__ __launch_bounds__(256) void window_attention_kernel(
    OT* __restrict__ out, const float* __restrict__ qkv, const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int* __restrict__ tok_pos, const int* __restrict__ tok_seq, const int* __restrict__ block_table, int items,
    int max_blocks, int num_blocks, int table_rows, int H, int G, int d, int dv, long ldq, long ldo, float scale, int window,
    int sink, const float* __restrict__ temp, const float* __restrict__ bias, int bias_rows, const float* __restrict__ sinkv,
    const float* __restrict__ gate, long ldg) {
  __shared__ float qs[4][kWinMaxD];
  const int wave = threadIdx.x >> 6, lane = lane_id();
  const int item = blockIdx.x * 4 + wave;
  if (item >= items) return;
  const int t = item / H, h = item % H, g = h / (H / G);
  const int pos = tok_pos[t], slot = tok_seq[t];
  OT* orow = out + (long)t * ldo + (long)h * dv;
  const bool live = slot >= 0 && slot < table_rows && pos >= 0 && pos / kWinBlock < max_blocks;
  if (!live) {                                   // padding row of a fixed-shape step
    for (int c = lane; c < dv; c += 64) orow[c] = (OT)0.f;
    return;
  }
  const float* qrow = qkv + (long)t * ldq + (long)h * d;
  const float hscale = temp ? scale * temp[h] : scale;
  for (int i = lane; i < d; i += 64) qs[wave][i] = qrow[i] * hscale;
  __builtin_amdgcn_wave_barrier();
  const int* table = block_table + (long)slot * max_blocks;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = sink ? (sinkv ? sinkv[h] : 0.f) : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[kWinMaxD / 64];
#pragma unroll
  for (int c = 0; c < kWinMaxD / 64; ++c) acc[c] = 0.f;
  const int ncol = (dv + 63) / 64;
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    int blk = -1;
    if (j <= pos) blk = table[j / kWinBlock];
    const bool valid = blk >= 0 && blk < num_blocks;
    float s = -INFINITY;
    if (valid) {
      const T* krow = kcache + (((long)blk * G + g) * kWinBlock + (j % kWinBlock)) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot += qs[wave][i] * (float)krow[i];
      if (bias) dot += bias[(long)min(pos - j, bias_rows - 1) * H + h];
      s = dot;
    }
    const float cm = wave_max(s);
    const float m_new = fmaxf(m, cm);
    if (m_new == -INFINITY) continue;             // no key of this step is readable (and no sink): nothing to add
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < kWinMaxD / 64; ++c) acc[c] *= corr;
    const int nk = (pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64;
    for (int jj = 0; jj < nk; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const int bj = __shfl(blk, jj, 64);
      if (pj == 0.f) continue;                    // (uniform over the wave: an unreadable key, or a weight that underflowed)
      const T* vrow = vcache + (((long)bj * G + g) * kWinBlock + ((j0 + jj) % kWinBlock)) * dv;
#pragma unroll
      for (int c = 0; c < kWinMaxD / 64; ++c)
        if (c < ncol) { const int col = c * 64 + lane; if (col < dv) acc[c] += pj * (float)vrow[col]; }
    }
  }
  float inv = l > 0.f ? 1.f / l : 0.f;
  if (gate) inv *= 1.f / (1.f + expf(-gate[(long)t * ldg + h]));
#pragma unroll
  for (int c = 0; c < kWinMaxD / 64; ++c)
    if (c < ncol) { const int col = c * 64 + lane; if (col < dv) orow[col] = (OT)(acc[c] * inv); }
}

// Value mixing on a bf16 fused q|k|v activation, ahead of the fragment-ordered cache write: the first mixing layer
// of a stack remembers its values for this step's tokens (mix 1), later ones blend theirs with them (mix 2), in fp32.
__global__ __launch_bounds__(256) void value_mix_kernel(bf16* __restrict__ qkv, float* __restrict__ vfirst,
                                                        const float* __restrict__ lam_p, int mix, int v_off, int v_cols, long ld) {
  const int t = blockIdx.x;
  bf16* row = qkv + (long)t * ld + v_off;
  float* vf = vfirst + (long)t * v_cols;
  const float lam = mix == 2 ? lam_p[0] : 0.f;
  for (int i = threadIdx.x; i < v_cols; i += 256) {
    const float v = (float)row[i];
    if (mix == 1) vf[i] = v;
    else row[i] = (bf16)((1.f - lam) * v + lam * vf[i]);
  }
}

}  // namespace dlia

extern "C" void dlia_value_mix(void* qkv, float* vfirst, const float* lam, int mix, int T, int v_off, int v_cols, long ld,
                               hipStream_t stream) {
  if (T <= 0 || mix == 0) return;
  hipLaunchKernelGGL(dlia::value_mix_kernel, dim3(T), dim3(256), 0, stream, (dlia::bf16*)qkv, vfirst, lam, mix, v_off, v_cols, ld);
}

extern "C" void dlia_kv_store(const float* qkv, float* vfirst, const float* lam, int mix, void* kcache, void* vcache,
                              int cache_f32, const int* tok_pos, const int* tok_seq, const int* block_table, int T,
                              int max_blocks, int num_blocks, int table_rows, int G, int d, int dv, int q_cols, long ld,
                              hipStream_t stream) {
  if (T <= 0) return;
  if (cache_f32)
    hipLaunchKernelGGL(dlia::kv_store_kernel<float>, dim3(T), dim3(256), 0, stream, qkv, vfirst, lam, mix, (float*)kcache,
                       (float*)vcache, tok_pos, tok_seq, block_table, max_blocks, num_blocks, table_rows, G, d, dv, q_cols, ld);
  else
    hipLaunchKernelGGL(dlia::kv_store_kernel<dlia::bf16>, dim3(T), dim3(256), 0, stream, qkv, vfirst, lam, mix,
                       (dlia::bf16*)kcache, (dlia::bf16*)vcache, tok_pos, tok_seq, block_table, max_blocks, num_blocks,
                       table_rows, G, d, dv, q_cols, ld);
}

extern "C" void dlia_window_attention(void* out, const float* qkv, const void* kcache, const void* vcache, int f32,
                                      const int* tok_pos, const int* tok_seq, const int* block_table, int T, int max_blocks,
                                      int num_blocks, int table_rows, int H, int G, int d, int dv, long ldq, long ldo,
                                      float scale, int window, int sink, const float* temp, const float* bias, int bias_rows,
                                      const float* sinkv, const float* gate, long ldg, hipStream_t stream) {
  const int items = T * H;
  if (items <= 0) return;
  const dim3 grid((items + 3) / 4);
  if (f32)
    hipLaunchKernelGGL((dlia::window_attention_kernel<float, float>), grid, dim3(256), 0, stream, (float*)out, qkv,
                       (const float*)kcache, (const float*)vcache, tok_pos, tok_seq, block_table, items, max_blocks, num_blocks,
                       table_rows, H, G, d, dv, ldq, ldo, scale, window, sink, temp, bias, bias_rows, sinkv, gate, ldg);
  else
    hipLaunchKernelGGL((dlia::window_attention_kernel<dlia::bf16, dlia::bf16>), grid, dim3(256), 0, stream, (dlia::bf16*)out, qkv,
                       (const dlia::bf16*)kcache, (const dlia::bf16*)vcache, tok_pos, tok_seq, block_table, items, max_blocks,
                       num_blocks, table_rows, H, G, d, dv, ldq, ldo, scale, window, sink, temp, bias, bias_rows, sinkv, gate, ldg);
}
