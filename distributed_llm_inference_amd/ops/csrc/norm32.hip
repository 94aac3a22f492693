// Kernels for models whose residual stream is kept in fp32: embedding gather into fp32 rows, and RMSNorm
// with fp32 statistics over fp32 rows whose output feeds a GEMM in the compute type (bf16 or fp32).
//
// The norm kernel covers the three places a sandwich-norm layer (a norm before AND after every sublayer)
// needs one, in one launch each:
//   plain     out = rms(x) * (off + w)                                   (first layer, final norm; rows may be gathered)
//   sandwich  x  += rms(y) * (off + wb);  out = rms(x) * (off + wn)      (post-norm of a sublayer, residual add, and the
//                                                                         pre-norm of the next sublayer)
//   closing   x  += rms(y) * (off + wb)                                  (after the last sublayer of the stage)
// `off` is 1 for weights stored as their distance from one, 0 for plain weights. One workgroup per row.
#include "common.h"
#include "launch.h"

namespace dlia {

constexpr int kN32Threads = 256;

template <typename T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return (T)v; }

template <typename TT>
__global__ __launch_bounds__(128) void embed32_kernel(float* __restrict__ out, const int* __restrict__ ids,
                                                      const TT* __restrict__ table, int H, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // never fault on a bad id
  const TT* src = table + (long)id * H;
  float* dst = out + (long)t * H;
  for (int i = threadIdx.x; i < H; i += 128) dst[i] = to_f32(src[i]);
}

template <typename OT>
__global__ __launch_bounds__(kN32Threads) void norm32_kernel(
    OT* __restrict__ out, float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ wb,
    const float* __restrict__ wn, const int* __restrict__ row_idx, int H, long ldx, long ldy, long ldo,
    float eps, float off) {
  __shared__ float scratch[16];
  const int orow = blockIdx.x;
  const long irow = row_idx ? row_idx[orow] : orow;
  float* xr = x + irow * ldx;
  if (y) {
    const float* yr = y + irow * ldy;
    float s = 0.f;
    for (int i = threadIdx.x; i < H; i += kN32Threads) { const float v = yr[i]; s += v * v; }
    s = block_sum(s, scratch);
    const float r = rsqrtf(s / H + eps);
    for (int i = threadIdx.x; i < H; i += kN32Threads) xr[i] += yr[i] * r * (off + wb[i]);
    // (each thread re-reads only the elements it wrote itself below: no barrier needed for visibility)
  }
  if (!out) return;
  float s = 0.f;
  for (int i = threadIdx.x; i < H; i += kN32Threads) { const float v = xr[i]; s += v * v; }
  s = block_sum(s, scratch);
  const float r = rsqrtf(s / H + eps);
  OT* outr = out + (long)orow * ldo;
  for (int i = threadIdx.x; i < H; i += kN32Threads) outr[i] = from_f32<OT>(xr[i] * r * (off + wn[i]));
}

// out[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * w[:] * silu(gate[t, h, :]): the read-out of a recurrent mixer, normalised
// per head and gated. One wave per (token, head).
template <typename OT>
__global__ __launch_bounds__(256) void gated_headnorm_kernel(OT* __restrict__ out, const float* __restrict__ o,
                                                             const float* __restrict__ gate, const float* __restrict__ w,
                                                             int items, int heads, int dv, long ldo_in, long ldg, long ld_out,
                                                             float eps) {
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const int t = item / heads, h = item % heads, lane = lane_id();
  const float* orow = o + (long)t * ldo_in + (long)h * dv;
  const float* grow = gate + (long)t * ldg + (long)h * dv;
  float s = 0.f;
  for (int i = lane; i < dv; i += 64) { const float v = orow[i]; s += v * v; }
  s = wave_sum(s);
  const float r = rsqrtf(s / dv + eps);
  OT* dst = out + (long)t * ld_out + (long)h * dv;
  for (int i = lane; i < dv; i += 64) {
    const float g = grow[i];
    dst[i] = from_f32<OT>(orow[i] * r * w[i] * (g / (1.f + expf(-g))));
  }
}

}  // namespace dlia

extern "C" void dlia_embed32(float* out, const int* ids, const void* table, int table_f32, int T, int H, int vocab,
                             hipStream_t stream) {
  if (T <= 0) return;
  if (table_f32)
    hipLaunchKernelGGL(dlia::embed32_kernel<float>, dim3(T), dim3(128), 0, stream, out, ids, (const float*)table, H, vocab);
  else
    hipLaunchKernelGGL(dlia::embed32_kernel<dlia::bf16>, dim3(T), dim3(128), 0, stream, out, ids, (const dlia::bf16*)table, H, vocab);
}

extern "C" void dlia_norm32(void* out, int out_f32, float* x, const float* y, const float* wb, const float* wn,
                            const int* row_idx, int rows, int H, long ldx, long ldy, long ldo, float eps, float off,
                            hipStream_t stream) {
  if (rows <= 0) return;
  if (out_f32 || !out)
    hipLaunchKernelGGL(dlia::norm32_kernel<float>, dim3(rows), dim3(dlia::kN32Threads), 0, stream, (float*)out, x, y, wb, wn,
                       row_idx, H, ldx, ldy, ldo, eps, off);
  else
    hipLaunchKernelGGL(dlia::norm32_kernel<dlia::bf16>, dim3(rows), dim3(dlia::kN32Threads), 0, stream, (dlia::bf16*)out, x, y,
                       wb, wn, row_idx, H, ldx, ldy, ldo, eps, off);
}

extern "C" void dlia_gated_headnorm(void* out, int out_f32, const float* o, const float* gate, const float* w, int T,
                                    int heads, int dv, long ldo_in, long ldg, long ld_out, float eps, hipStream_t stream) {
  const int items = T * heads;
  if (items <= 0) return;
  if (out_f32)
    hipLaunchKernelGGL(dlia::gated_headnorm_kernel<float>, dim3((items + 3) / 4), dim3(256), 0, stream, (float*)out, o, gate, w,
                       items, heads, dv, ldo_in, ldg, ld_out, eps);
  else
    hipLaunchKernelGGL(dlia::gated_headnorm_kernel<dlia::bf16>, dim3((items + 3) / 4), dim3(256), 0, stream, (dlia::bf16*)out,
                       o, gate, w, items, heads, dv, ldo_in, ldg, ld_out, eps);
}
