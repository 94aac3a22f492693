// Routed feed-forward (mixture of experts) without a host round trip: routing, a plan that sorts the step's (token, choice)
// pairs by expert into 16-row tiles, the experts' two GEMMs over those tiles, and the weighted sum per token.
//
//   moe_route    one thread per token. Scores are sigmoids of the fp32 router logits. Experts form `groups` equal groups of
//                neighbours; a group's score is the sum of its two largest scores; the `keep` best groups stay; the `top`
//                best experts of those are chosen (equal scores: the lower index), weighted score / (sum + 1e-20) * scale.
//   moe_plan     one workgroup. Counts the pairs per expert, lays the experts' row ranges out one after the other, each
//                padded to whole 16-row tiles, and writes for every padded row its token (or -1), for every pair its row,
//                for every tile its expert; tiles[0] holds the number of tiles. Rows of one expert are in no fixed order:
//                every row is computed on its own, so the order does not reach the results.
//   moe_up       grid (column blocks, tiles): act[row, f] = g s(1.702 g) (u + 1), g = min(x . Wg[e][f], limit),
//                u = clamp(x . Wu[e][f], -limit, limit), x the row's token. One wave per 16 columns, gate and up in two
//                accumulators over the same A fragments.
//   moe_down     y[row, c] = act[row] . Wd[e][c] in fp32.
//   moe_combine  out[t, :] = sum over the token's choices of weight * y[row, :], in the order of the choices (fp32).
// Operands are bf16 (16x16x32 MFMA) or fp32 (16x16x4 MFMA, true 32-bit), fragments read straight from the K-contiguous rows.
#include "common.h"
#include "frag.h"
#include "launch.h"

namespace dlia {

constexpr int kMoeMaxExperts = 256;

__global__ __launch_bounds__(64) void moe_route_kernel(int* __restrict__ sel, float* __restrict__ wts,
                                                       const float* __restrict__ logits, long ld, int T, int E, int top,
                                                       int groups, int keep, float scale) {
  const int t = blockIdx.x * 64 + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (long)t * ld;
  const int per = E / groups;
  auto score = [&](int e) { return 1.f / (1.f + expf(-z[e])); };
  // the groups that stay: `keep` times the best group not yet taken
  unsigned long long gmask[4] = {0ull, 0ull, 0ull, 0ull};
  for (int r = 0; r < keep; ++r) {
    int best = -1; float bs = -1.f;
    for (int g = 0; g < groups; ++g) {
      if (gmask[g >> 6] >> (g & 63) & 1ull) continue;
      float a = -1.f, b = -1.f;                       // the two largest scores of the group
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float s = score(e);
        if (s > a) { b = a; a = s; } else if (s > b) b = s;
      }
      const float gs = a + (b > 0.f ? b : 0.f);
      if (gs > bs) { bs = gs; best = g; }
    }
    if (best >= 0) gmask[best >> 6] |= 1ull << (best & 63);
  }
  unsigned long long emask[4] = {0ull, 0ull, 0ull, 0ull};
  float total = 0.f;
  for (int r = 0; r < top; ++r) {
    int best = 0; float bs = -1.f;
    for (int e = 0; e < E; ++e) {
      const int g = e / per;
      if (!(gmask[g >> 6] >> (g & 63) & 1ull) || (emask[e >> 6] >> (e & 63) & 1ull)) continue;
      const float s = score(e);
      if (s > bs) { bs = s; best = e; }
    }
    emask[best >> 6] |= 1ull << (best & 63);
    sel[(long)t * top + r] = best;
    wts[(long)t * top + r] = bs;
    total += bs;
  }
  const float inv = scale / (total + 1e-20f);
  for (int r = 0; r < top; ++r) wts[(long)t * top + r] *= inv;
}

// tiles: [0] number of tiles, [1 + i] expert of tile i. row_tok [max_rows], pair_row [T * top].
__global__ __launch_bounds__(1024) void moe_plan_kernel(int* __restrict__ tiles, int* __restrict__ row_tok,
                                                        int* __restrict__ pair_row, const int* __restrict__ sel, int pairs,
                                                        int top, int E, int max_rows) {
  __shared__ int count[kMoeMaxExperts], start[kMoeMaxExperts], fill[kMoeMaxExperts];
  __shared__ int ntiles;
  for (int e = threadIdx.x; e < E; e += 1024) { count[e] = 0; fill[e] = 0; }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024) atomicAdd(&count[sel[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      const int n = (count[e] + 15) / 16;
      for (int i = 0; i < n; ++i) tiles[1 + nt + i] = e;
      nt += n; at += n * 16;
    }
    tiles[0] = nt;
    ntiles = nt;
  }
  __syncthreads();
  const int used = ntiles * 16;
  for (int i = threadIdx.x; i < max_rows; i += 1024) row_tok[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024) {
    const int e = sel[i];
    const int r = start[e] + atomicAdd(&fill[e], 1);
    if (r < max_rows && r < used) { row_tok[r] = i / top; pair_row[i] = r; }
  }
}

template <typename T, typename OT>
__global__ __launch_bounds__(256) void moe_up_kernel(OT* __restrict__ act, const T* __restrict__ x, const T* __restrict__ wg,
                                                     const T* __restrict__ wu, const int* __restrict__ tiles,
                                                     const int* __restrict__ row_tok, int F, int K, long ldx, long lda,
                                                     float limit, int vec_ok) {
  constexpr int VEC = 16 / sizeof(T), KS = 4 * VEC;
  const int tile = blockIdx.y;
  if (tile >= tiles[0]) return;
  const int e = tiles[1 + tile];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int f0 = blockIdx.x * 64 + wave * 16;
  if (f0 >= F) return;
  const int tok = row_tok[tile * 16 + r16];
  const bool av = tok >= 0, wv = f0 + r16 < F;
  const T* arow = x + (long)(av ? tok : 0) * ldx;
  const long wrow = ((long)e * F + (wv ? f0 + r16 : 0)) * K;
  f32x4 ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += KS) {
    const int k = k0 + kq * VEC;
    const u32x4 a = load_frag<T>(arow, k, K, av, vec_ok);
    ag = mma_frag(T{}, a, load_frag<T>(wg + wrow, k, K, wv, vec_ok), ag);
    au = mma_frag(T{}, a, load_frag<T>(wu + wrow, k, K, wv, vec_ok), au);
  }
  if (!wv) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = tile * 16 + kq * 4 + r;
    const float g = fminf(ag[r], limit), u = fminf(fmaxf(au[r], -limit), limit);
    act[(long)row * lda + f0 + r16] = (OT)(g / (1.f + expf(-1.702f * g)) * (u + 1.f));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(float* __restrict__ y, const T* __restrict__ act, const T* __restrict__ wd,
                                                       const int* __restrict__ tiles, const int* __restrict__ row_tok,
                                                       int H, int F, long lda, int vec_ok) {
  constexpr int VEC = 16 / sizeof(T), KS = 4 * VEC;
  const int tile = blockIdx.y;
  if (tile >= tiles[0]) return;
  const int e = tiles[1 + tile];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int c0 = blockIdx.x * 64 + wave * 16;
  if (c0 >= H) return;
  const bool av = row_tok[tile * 16 + r16] >= 0, wv = c0 + r16 < H;
  const T* arow = act + (long)(tile * 16 + r16) * lda;
  const T* wrow = wd + ((long)e * H + (wv ? c0 + r16 : 0)) * F;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < F; k0 += KS) {
    const int k = k0 + kq * VEC;
    acc = mma_frag(T{}, load_frag<T>(arow, k, F, av, vec_ok), load_frag<T>(wrow, k, F, wv, vec_ok), acc);
  }
  if (!wv) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) y[(long)(tile * 16 + kq * 4 + r) * H + c0 + r16] = acc[r];
}

__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y,
                                                          const int* __restrict__ pair_row, const float* __restrict__ wts,
                                                          int H, int top, long ldo) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < H; c += 256) {
    float s = 0.f;
    for (int r = 0; r < top; ++r) s += wts[(long)t * top + r] * y[(long)pair_row[(long)t * top + r] * H + c];
    out[(long)t * ldo + c] = s;
  }
}

}  // namespace dlia

extern "C" void dlia_moe_route(int* sel, float* wts, const float* logits, long ld, int T, int E, int top, int groups, int keep,
                               float scale, hipStream_t stream) {
  if (T <= 0) return;
  hipLaunchKernelGGL(dlia::moe_route_kernel, dim3((T + 63) / 64), dim3(64), 0, stream, sel, wts, logits, ld, T, E, top, groups,
                     keep, scale);
}

extern "C" void dlia_moe_plan(int* tiles, int* row_tok, int* pair_row, const int* sel, int pairs, int top, int E, int max_rows,
                              hipStream_t stream) {
  hipLaunchKernelGGL(dlia::moe_plan_kernel, dim3(1), dim3(1024), 0, stream, tiles, row_tok, pair_row, sel, pairs, top, E, max_rows);
}

extern "C" void dlia_moe_up(void* act, const void* x, const void* wg, const void* wu, int f32, const int* tiles, const int* row_tok,
                            int max_tiles, int F, int K, long ldx, long lda, float limit, hipStream_t stream) {
  if (max_tiles <= 0) return;
  const dim3 grid((F + 63) / 64, max_tiles);
  if (f32) {
    const int ok = K % 4 == 0 && ldx % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)wg % 16 == 0 && (uintptr_t)wu % 16 == 0;
    hipLaunchKernelGGL((dlia::moe_up_kernel<float, float>), grid, dim3(256), 0, stream, (float*)act, (const float*)x,
                       (const float*)wg, (const float*)wu, tiles, row_tok, F, K, ldx, lda, limit, ok);
  } else {
    const int ok = K % 8 == 0 && ldx % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)wg % 16 == 0 && (uintptr_t)wu % 16 == 0;
    hipLaunchKernelGGL((dlia::moe_up_kernel<dlia::bf16, dlia::bf16>), grid, dim3(256), 0, stream, (dlia::bf16*)act,
                       (const dlia::bf16*)x, (const dlia::bf16*)wg, (const dlia::bf16*)wu, tiles, row_tok, F, K, ldx, lda, limit, ok);
  }
}

extern "C" void dlia_moe_down(float* y, const void* act, const void* wd, int f32, const int* tiles, const int* row_tok,
                              int max_tiles, int H, int F, long lda, hipStream_t stream) {
  if (max_tiles <= 0) return;
  const dim3 grid((H + 63) / 64, max_tiles);
  if (f32) {
    const int ok = F % 4 == 0 && lda % 4 == 0 && (uintptr_t)act % 16 == 0 && (uintptr_t)wd % 16 == 0;
    hipLaunchKernelGGL(dlia::moe_down_kernel<float>, grid, dim3(256), 0, stream, y, (const float*)act, (const float*)wd, tiles,
                       row_tok, H, F, lda, ok);
  } else {
    const int ok = F % 8 == 0 && lda % 8 == 0 && (uintptr_t)act % 16 == 0 && (uintptr_t)wd % 16 == 0;
    hipLaunchKernelGGL(dlia::moe_down_kernel<dlia::bf16>, grid, dim3(256), 0, stream, y, (const dlia::bf16*)act,
                       (const dlia::bf16*)wd, tiles, row_tok, H, F, lda, ok);
  }
}

extern "C" void dlia_moe_combine(float* out, const float* y, const int* pair_row, const float* wts, int T, int H, int top, long ldo,
                                 hipStream_t stream) {
  if (T <= 0) return;
  hipLaunchKernelGGL(dlia::moe_combine_kernel, dim3(T), dim3(256), 0, stream, out, y, pair_row, wts, H, top, ldo);
}
