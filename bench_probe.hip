// Benchmark-only device probes (built into libbench_probe.so next to bench.py; not part of the
// product library or its header).  They give bench.py the ceilings it prints beside the
// attention and merge kernels:
//   bench_probe_mfma   sustained rate of back-to-back v_mfma_f32_32x32x16_bf16 from registers
//                      only, on the operand bits it is given.  The shader clock of this part
//                      follows the power drawn and the matrix pipe's power follows the bit
//                      activity of its operands, so random operands give the practical ceiling
//                      of any bf16 MFMA kernel fed with ordinary data.
//   bench_stream_mix   n_src streams read and one written with 16-byte accesses, the access
//                      shape of the merge kernel: the device's rate for that read:write mix.
//   bench_atomic_rate  device-wide rate of L2 atomics (fp32 add, u32 add, f64 add) and of plain dword
//                      stores with the access shape a backward that sums dQ with atomics would have
//                      (a wave instruction covers two 128-byte lines): the figure that decides
//                      between recomputing S and dP in a second kernel and one fused kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__global__ __launch_bounds__(256) void probe_mfma_kernel(const u32x4* in, float* out, int iters) {
  const u32x4 ra = in[threadIdx.x], rb = in[256 + threadIdx.x];
  bf16x8 a, b;
  __builtin_memcpy(&a, &ra, 16);
  __builtin_memcpy(&b, &rb, 16);
  f32x16 c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = f32x16{0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += c[i][j];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Same loop, but every MFMA takes a different pair of operand fragments (8 A x 8 B fragments cycled
// from registers), as a real GEMM does: the operand latches of the matrix pipe then toggle on every
// instruction, which the loop above (one A, one B for ever) does not exercise.
__global__ __launch_bounds__(256) void probe_mfma_rot_kernel(const u32x4* in, float* out, int iters) {
  bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const u32x4 ra = in[(2 * i) * 256 + threadIdx.x], rb = in[(2 * i + 1) * 256 + threadIdx.x];
    __builtin_memcpy(&a[i], &ra, 16);
    __builtin_memcpy(&b[i], &rb, 16);
  }
  f32x16 c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = f32x16{0};
  for (int it = 0; it < iters; it += 8) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) c[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + i) & 7], b[(u + 3 * i) & 7], c[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += c[i][j];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

template <int MODE>
__global__ __launch_bounds__(256) void atomic_rate_kernel(void* buf, int64_t n_dwords, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t base = ((int64_t)blockIdx.x * 4 + wave) * 64 * 64;      // each wave walks its own region
  for (int it = 0; it < iters; ++it) {
    const int64_t off = (base + (int64_t)it * 64 + lane) % n_dwords;
    if (MODE == 0) __builtin_amdgcn_global_atomic_fadd_f32((__attribute__((address_space(1))) float*)buf + off, 1.0f);
    if (MODE == 1) atomicAdd((unsigned*)buf + off, 1u);
    if (MODE == 2) atomicAdd((double*)buf + (off >> 1), 1.0);
    if (MODE == 3) ((volatile unsigned*)buf)[off] = 1u;
  }
}

constexpr int kMaxSrc = 8;
struct MixParams {
  const u32x4* src[kMaxSrc];
  u32x4* dst;
  int64_t n_chunks;      // 16-byte chunks per stream
};

// Each thread keeps N * kUnroll 16-byte loads in flight, combines them with one xor per word
// and writes one 16-byte chunk per kUnroll group: the merge kernel's memory pattern without
// its arithmetic.
template <int N, bool kNonTemporal>
__global__ __launch_bounds__(256) void stream_mix_kernel(const MixParams p) {
  constexpr int kUnroll = 4;
  const int64_t stride = (int64_t)gridDim.x * 256 * kUnroll;
  for (int64_t c0 = ((int64_t)blockIdx.x * kUnroll) * 256 + threadIdx.x; c0 < p.n_chunks; c0 += stride) {
    u32x4 v[kUnroll][N];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t c = c0 + u * 256;
      if (c < p.n_chunks) {
#pragma unroll
        for (int i = 0; i < N; ++i)
          v[u][i] = kNonTemporal ? __builtin_nontemporal_load(p.src[i] + c) : p.src[i][c];
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t c = c0 + u * 256;
      if (c >= p.n_chunks) break;
      u32x4 acc = v[u][0];
#pragma unroll
      for (int i = 1; i < N; ++i) acc ^= v[u][i];
      if (kNonTemporal) __builtin_nontemporal_store(acc, p.dst + c);
      else p.dst[c] = acc;
    }
  }
}

template <int N>
static int launch_mix(const MixParams& p, int blocks, int non_temporal, hipStream_t st) {
  if (non_temporal) hipLaunchKernelGGL((stream_mix_kernel<N, true>), dim3(blocks), dim3(256), 0, st, p);
  else              hipLaunchKernelGGL((stream_mix_kernel<N, false>), dim3(blocks), dim3(256), 0, st, p);
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

extern "C" int bench_probe_mfma(const void* operands, float* out, int n_blocks, int iters, void* stream) {
  if (!operands || !out) return -1;
  if (n_blocks <= 0 || iters <= 0) return -2;
  if (reinterpret_cast<uintptr_t>(operands) & 15) return -4;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(n_blocks), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4*)operands, out, iters);
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

// operands: 16 x 256 x 16 bytes (8 A and 8 B fragments per thread, interleaved A0 B0 A1 B1 ...);
// iters is rounded up to a multiple of 8.
extern "C" int bench_probe_mfma_rotating(const void* operands, float* out, int n_blocks, int iters, void* stream) {
  if (!operands || !out) return -1;
  if (n_blocks <= 0 || iters <= 0) return -2;
  if (reinterpret_cast<uintptr_t>(operands) & 15) return -4;
  hipLaunchKernelGGL(probe_mfma_rot_kernel, dim3(n_blocks), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4*)operands, out, iters);
  return hipGetLastError() == hipSuccess ? 0 : -6;
}

// srcs: HOST array of n_src DEVICE pointers (16-byte aligned, n_bytes each); dst likewise.
extern "C" int bench_stream_mix(const void* const* srcs, int n_src, void* dst, int64_t n_bytes,
                                int n_blocks, int non_temporal, void* stream) {
  if (!srcs || !dst) return -1;
  if (n_src < 1 || n_src > kMaxSrc || n_bytes <= 0 || n_bytes % 16 || n_blocks <= 0) return -2;
  MixParams p;
  for (int i = 0; i < kMaxSrc; ++i) {
    p.src[i] = i < n_src ? (const u32x4*)srcs[i] : nullptr;
    if (i < n_src && (!srcs[i] || (reinterpret_cast<uintptr_t>(srcs[i]) & 15))) return -4;
  }
  if (reinterpret_cast<uintptr_t>(dst) & 15) return -4;
  p.dst = (u32x4*)dst;
  p.n_chunks = n_bytes / 16;
  hipStream_t st = (hipStream_t)stream;
  switch (n_src) {
    case 1: return launch_mix<1>(p, n_blocks, non_temporal, st);
    case 2: return launch_mix<2>(p, n_blocks, non_temporal, st);
    case 3: return launch_mix<3>(p, n_blocks, non_temporal, st);
    case 4: return launch_mix<4>(p, n_blocks, non_temporal, st);
    case 5: return launch_mix<5>(p, n_blocks, non_temporal, st);
    case 6: return launch_mix<6>(p, n_blocks, non_temporal, st);
    case 7: return launch_mix<7>(p, n_blocks, non_temporal, st);
    default: return launch_mix<8>(p, n_blocks, non_temporal, st);
  }
}

// mode: 0 fp32 atomic add (no return), 1 u32 atomic add, 2 f64 atomic add, 3 plain dword store.
// n_blocks x 256 threads, each issuing `iters` operations on buf[0 .. n_dwords) (device, 8-byte aligned).
extern "C" int bench_atomic_rate(void* buf, int64_t n_dwords, int mode, int n_blocks, int iters, void* stream) {
  if (!buf) return -1;
  if (n_dwords < 4096 || n_dwords % 2 || n_blocks <= 0 || iters <= 0 || mode < 0 || mode > 3) return -2;
  hipStream_t st = (hipStream_t)stream;
  switch (mode) {
    case 0: hipLaunchKernelGGL(atomic_rate_kernel<0>, dim3(n_blocks), dim3(256), 0, st, buf, n_dwords, iters); break;
    case 1: hipLaunchKernelGGL(atomic_rate_kernel<1>, dim3(n_blocks), dim3(256), 0, st, buf, n_dwords, iters); break;
    case 2: hipLaunchKernelGGL(atomic_rate_kernel<2>, dim3(n_blocks), dim3(256), 0, st, buf, n_dwords, iters); break;
    default: hipLaunchKernelGGL(atomic_rate_kernel<3>, dim3(n_blocks), dim3(256), 0, st, buf, n_dwords, iters); break;
  }
  return hipGetLastError() == hipSuccess ? 0 : -6;
}
