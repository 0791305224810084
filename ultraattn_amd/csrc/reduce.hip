// Gradient reductions across partial results: HBM-bandwidth bound streaming kernels.
//
//  grad_accumulate_kernel : one step of a running fp32 sum, acc += partial, with the bf16 rounding
//                           of the sum written in the same pass (the accumulation of
//                           ring_flash_attn/ring_flash_attn.py:110-118: partial gradients are added
//                           into fp32 buffers and cast once).
//  grad_sum_kernel        : out = bf16(scale * sum_p part_p) over n_parts partial gradients, fp32 or
//                           bf16, in one pass; the output may be strided by (batch, token, head).
#include <algorithm>
#include "ua_common.h"

namespace ua {

constexpr int kRedThreads = 256;
constexpr int kRedBlocks = 8192;         // grid cap of the sum: 32 workgroups per CU, grid-stride beyond

__device__ __forceinline__ void unpack8(const u32x4 r, float (&x)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) { x[2 * j] = __uint_as_float(r[j] << 16); x[2 * j + 1] = __uint_as_float(r[j] & 0xffff0000u); }
}
__device__ __forceinline__ bf16x8 pack8(const float (&x)[8]) {
  bf16x8 w;
#pragma unroll
  for (int j = 0; j < 8; ++j) w[j] = (bf16)x[j];
  return w;
}

// mode 0: acc += partial, out = bf16(acc) when out != NULL
// mode 1: acc  = float(out) + partial, out = bf16(acc)          (first step of a chain)
// mode 2: out  = bf16(float(out) + partial)                     (no fp32 accumulator)
template <int kMode>
__global__ __launch_bounds__(kRedThreads) void grad_accumulate_kernel(float* acc, const bf16* partial, bf16* out, int64_t n_chunks) {
  // kVec chunks of 8 elements per thread and step, every load of the step issued before the first use
  constexpr int kVec = 4;
  const int64_t stride = (int64_t)gridDim.x * kRedThreads * kVec;
  for (int64_t c0 = (int64_t)blockIdx.x * kRedThreads * kVec + threadIdx.x; c0 < n_chunks; c0 += stride) {
    u32x4 py[kVec], po[kVec];
    f32x4 a0[kVec], a1[kVec];
#pragma unroll
    for (int u = 0; u < kVec; ++u) {
      const int64_t c = c0 + u * kRedThreads;
      if (c >= n_chunks) break;
      py[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(partial) + c);
      if (kMode == 0) {
        a0[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(acc) + 2 * c);
        a1[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(acc) + 2 * c + 1);
      } else {
        po[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(out) + c);
      }
    }
#pragma unroll
    for (int u = 0; u < kVec; ++u) {
      const int64_t c = c0 + u * kRedThreads;
      if (c >= n_chunks) break;
      float x[8], y[8];
      unpack8(py[u], y);
      if (kMode == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) { x[j] = a0[u][j]; x[4 + j] = a1[u][j]; }
      } else {
        unpack8(po[u], x);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += y[j];
      if (kMode != 2) {
        __builtin_nontemporal_store(f32x4{x[0], x[1], x[2], x[3]}, reinterpret_cast<f32x4*>(acc) + 2 * c);
        __builtin_nontemporal_store(f32x4{x[4], x[5], x[6], x[7]}, reinterpret_cast<f32x4*>(acc) + 2 * c + 1);
      }
      if (out) __builtin_nontemporal_store(pack8(x), reinterpret_cast<bf16x8*>(out) + c);
    }
  }
}

struct SumParams {
  const void* parts[UA_MAX_PARTS];
  bf16* out;
  int n_parts, seqlen, n_heads;
  Strides3 os;
  float scale;
  int64_t n_chunks;        // batch * seqlen * n_heads * 16
};

template <bool kF32>
__global__ __launch_bounds__(kRedThreads) void grad_sum_kernel(const SumParams p) {
  for (int64_t c = (int64_t)blockIdx.x * kRedThreads + threadIdx.x; c < p.n_chunks; c += (int64_t)gridDim.x * kRedThreads) {
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = 0.f;
    for (int i = 0; i < p.n_parts; ++i) {
      if (kF32) {
        const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.parts[i]) + 2 * c);
        const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.parts[i]) + 2 * c + 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) { x[j] += a[j]; x[4 + j] += b[j]; }
      } else {
        float y[8];
        unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.parts[i]) + c), y);
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] += y[j];
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] *= p.scale;
    const int64_t row = c >> 4;
    const int h = (int)(row % p.n_heads);
    const int64_t t = row / p.n_heads;
    const int64_t s = t % p.seqlen, b = t / p.seqlen;
    *reinterpret_cast<bf16x8*>(p.out + b * p.os.b + s * p.os.s + h * p.os.h + (c & 15) * 8) = pack8(x);
  }
}

// Shared by ua_grad_sum and the split dense backward: the parts are contiguous [batch, seqlen,
// n_heads, 128] arrays, the output takes (batch, token, head) element strides.
int launch_grad_sum(const void* const* parts, int n_parts, bool parts_fp32, void* out, const int64_t* out_strides,
                    int batch, int seqlen, int n_heads, float scale, hipStream_t st) {
  SumParams p;
  for (int i = 0; i < UA_MAX_PARTS; ++i) p.parts[i] = i < n_parts ? parts[i] : nullptr;
  p.out = (bf16*)out; p.n_parts = n_parts; p.seqlen = seqlen; p.n_heads = n_heads;
  p.os = {out_strides[0], out_strides[1], out_strides[2]};
  p.scale = scale;
  p.n_chunks = (int64_t)batch * seqlen * n_heads * 16;
  const int blocks = (int)std::min<int64_t>((p.n_chunks + kRedThreads - 1) / kRedThreads, kRedBlocks);
  if (parts_fp32) hipLaunchKernelGGL(grad_sum_kernel<true>, dim3(blocks), dim3(kRedThreads), 0, st, p);
  else            hipLaunchKernelGGL(grad_sum_kernel<false>, dim3(blocks), dim3(kRedThreads), 0, st, p);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

}  // namespace ua

extern "C" int ua_grad_accumulate(float* acc, const void* partial, void* out, int64_t n, int init_from_out, void* stream) {
  using namespace ua;
  if (!partial || (!acc && !out) || (init_from_out && (!acc || !out))) return UA_ERR_NULL;
  if (n <= 0) return UA_ERR_SHAPE;
  if (n % 8 != 0 || !aligned16(partial) || (acc && !aligned16(acc)) || (out && !aligned16(out))) return UA_ERR_ALIGN;
  if (int rc = check_device()) return rc;
  const int64_t n_chunks = n / 8;
  const int blocks = (int)std::min<int64_t>((n_chunks + 4 * kRedThreads - 1) / (4 * kRedThreads), 4 * kRedBlocks);
  hipStream_t st = (hipStream_t)stream;
  if (!acc)               hipLaunchKernelGGL(grad_accumulate_kernel<2>, dim3(blocks), dim3(kRedThreads), 0, st, acc, (const bf16*)partial, (bf16*)out, n_chunks);
  else if (init_from_out) hipLaunchKernelGGL(grad_accumulate_kernel<1>, dim3(blocks), dim3(kRedThreads), 0, st, acc, (const bf16*)partial, (bf16*)out, n_chunks);
  else                    hipLaunchKernelGGL(grad_accumulate_kernel<0>, dim3(blocks), dim3(kRedThreads), 0, st, acc, (const bf16*)partial, (bf16*)out, n_chunks);
  return hipGetLastError() == hipSuccess ? UA_OK : UA_ERR_LAUNCH;
}

extern "C" int ua_grad_sum(const void* const* parts, int n_parts, int parts_fp32, void* out,
                           int batch, int seqlen, int n_heads, int head_dim, const int64_t* out_strides,
                           float scale, void* stream) {
  using namespace ua;
  if (!parts || !out || !out_strides) return UA_ERR_NULL;
  if (n_parts < 1 || n_parts > UA_MAX_PARTS || head_dim != kHeadDim) return UA_ERR_UNSUPPORTED;
  if (batch <= 0 || seqlen <= 0 || n_heads <= 0) return UA_ERR_SHAPE;
  if (!aligned16(out) || !strides_ok(out_strides)) return UA_ERR_ALIGN;
  for (int i = 0; i < n_parts; ++i) {
    if (!parts[i]) return UA_ERR_NULL;
    if (!aligned16(parts[i])) return UA_ERR_ALIGN;
  }
  if (int rc = check_device()) return rc;
  return launch_grad_sum(parts, n_parts, parts_fp32 != 0, out, out_strides, batch, seqlen, n_heads, scale, (hipStream_t)stream);
}
