// Benchmark-only device probes (built into libbench_probe.so next to bench.py; not part of the
// product library or its header).  They give bench.py the ceilings it prints beside the
// attention and merge kernels:
//   bench_probe_mfma   sustained rate of back-to-back v_mfma_f32_32x32x16_bf16 from registers
//                      only, on the operand bits it is given.  The shader clock of this part
//                      follows the power drawn and the matrix pipe's power follows the bit
//                      activity of its operands, so random operands give the practical ceiling
//                      of any bf16 MFMA kernel fed with ordinary data.
//   bench_probe_mfma_rotating / bench_probe_mfma16_rotating: the same with operands that change on every
//                      instruction, for v_mfma_f32_32x32x16_bf16 and v_mfma_f32_16x16x32_bf16; with 256 or 512
//                      workgroups of 4 waves (1 or 2 waves per SIMD) they give the device's ceiling rather than
//                      one instruction's at one occupancy.
//   bench_stream_mix   n_src streams read and one written with 16-byte accesses, the access
//                      shape of the merge kernel: the device's rate for that read:write mix.
//   bench_atomic_rate  device-wide rate of L2 atomics (fp32 add, u32 add, f64 add) and of plain dword
//                      stores with the access shape a backward that sums dQ with atomics would have
//                      (a wave instruction covers two 128-byte lines): the figure that decides
//                      between recomputing S and dP in a second kernel and one fused kernel.
//   bench_issue_mix    one loop iteration = 16 MFMAs plus the vector and LDS instructions that the forward kernel
//                      issues per 32 keys (40 fma-class, 16 exp2, 8 ds_read_b128, 16 ds_read_b64_tr_b16), on zero
//                      data, registers and LDS only, 1 or 2 waves per SIMD: time of the bare MFMA loop / time of a
//                      mix = the matrix-pipe occupancy that this instruction mix allows before barriers, copies
//                      and power come in.
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

// The other dense bf16 instruction, v_mfma_f32_16x16x32_bf16 (16384 flop, 4 accumulator registers), with
// rotating operands: 8 independent accumulators, 8 A x 8 B fragments cycled.
typedef __attribute__((ext_vector_type(4))) float f32x4;
__global__ __launch_bounds__(256) void probe_mfma16_rot_kernel(const u32x4* in, float* out, int iters) {
  bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const u32x4 ra = in[(2 * i) * 256 + threadIdx.x], rb = in[(2 * i + 1) * 256 + threadIdx.x];
    __builtin_memcpy(&a[i], &ra, 16);
    __builtin_memcpy(&b[i], &rb, 16);
  }
  f32x4 c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) c[i] = f32x4{0};
  for (int it = 0; it < iters; it += 8) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) c[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(u + i) & 7], b[(u + 3 * i) & 7], c[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) s += c[i][j];
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

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
// M MFMAs per iteration; per MFMA slot V/M fma, X/M exp2 interleaved behind it; L 128-bit and T transposing
// 64-bit LDS reads issued at the top of the iteration and consumed at its end.
template <int M, int V, int X, int L, int T>
__global__ __launch_bounds__(512) void issue_mix_kernel(float* out, int iters, float kk) {
  __shared__ __attribute__((aligned(1024))) unsigned char lds[32768];
  typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
  for (int i = threadIdx.x; i < 8192; i += blockDim.x) reinterpret_cast<uint32_t*>(lds)[i] = 0;
  __syncthreads();
  f32x16 c[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) c[i] = f32x16{0};
  const bf16x8 a = {0}, b = {0};
  float r[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = kk * threadIdx.x;
  const int lane = threadIdx.x & 63;
  constexpr int N = M > 0 ? M : 16;
  constexpr int VS = (V + N - 1) / N, XS = (X + N - 1) / N;
  for (int it = 0; it < iters; ++it) {
    u32x4 lv[L > 0 ? L : 1];
    bf16x4 tv[T > 0 ? T : 1];
#pragma unroll
    for (int j = 0; j < L; ++j) lv[j] = *reinterpret_cast<const u32x4*>(lds + lane * 16 + (j & 15) * 1024);
#pragma unroll
    for (int j = 0; j < T; ++j) tv[j] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(lds + lane * 8 + (j & 31) * 512));
    if (L + T > 0) __builtin_amdgcn_sched_group_barrier(0x100, L + T, 0);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (M > 0) c[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[i & 3], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < VS; ++j) if (i * VS + j < V) r[(i + j) & 7] = __builtin_fmaf(r[(i + j) & 7], kk, kk);
#pragma unroll
      for (int j = 0; j < XS; ++j) if (i * XS + j < X) r[(i + j + 4) & 7] = __builtin_amdgcn_exp2f(r[(i + j + 4) & 7]);
      if (M > 0) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (V + X > 0) __builtin_amdgcn_sched_group_barrier(0x002, VS + XS, 0);
    }
    uint32_t acc = 0;
#pragma unroll
    for (int j = 0; j < L; ++j) acc ^= lv[j][0] ^ lv[j][3];
#pragma unroll
    for (int j = 0; j < T; ++j) acc ^= __builtin_bit_cast(uint32_t, __builtin_shufflevector(tv[j], tv[j], 0, 1));
    if (L + T > 0) r[0] += __builtin_bit_cast(float, acc);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += c[i][j];
#pragma unroll
  for (int i = 0; i < 8; ++i) s += r[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
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

// Same operand layout as bench_probe_mfma_rotating; every thread issues 8 x iters (rounded up to a multiple
// of 8) v_mfma_f32_16x16x32_bf16.
extern "C" int bench_probe_mfma16_rotating(const void* operands, float* out, int n_blocks, int iters, void* stream) {
  if (!operands || !out) return -1;
  if (n_blocks <= 0 || iters <= 0) return -2;
  if (reinterpret_cast<uintptr_t>(operands) & 15) return -4;
  hipLaunchKernelGGL(probe_mfma16_rot_kernel, dim3(n_blocks), dim3(256), 0, (hipStream_t)stream,
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

// mix: 0 = 16 MFMA; 1 = + 40 fma + 16 exp2; 2 = 16 MFMA + 8 ds_read_b128 + 16 ds_read_b64_tr_b16; 3 = all of them;
// 4 = the vector work alone; 5 = the LDS reads alone.  waves_per_simd 1 or 2 (256 or 512 threads per workgroup, one
// workgroup per CU when n_blocks = number of CUs).  out: n_blocks x 512 floats.
extern "C" int bench_issue_mix(float* out, int n_blocks, int waves_per_simd, int mix, int iters, void* stream) {
  if (!out) return -1;
  if (n_blocks <= 0 || iters <= 0 || (waves_per_simd != 1 && waves_per_simd != 2) || mix < 0 || mix > 5) return -2;
  const dim3 g(n_blocks), t(256 * waves_per_simd);
  hipStream_t st = (hipStream_t)stream;
  switch (mix) {
    case 0: hipLaunchKernelGGL((issue_mix_kernel<16, 0, 0, 0, 0>), g, t, 0, st, out, iters, 0.f); break;
    case 1: hipLaunchKernelGGL((issue_mix_kernel<16, 40, 16, 0, 0>), g, t, 0, st, out, iters, 0.f); break;
    case 2: hipLaunchKernelGGL((issue_mix_kernel<16, 0, 0, 8, 16>), g, t, 0, st, out, iters, 0.f); break;
    case 3: hipLaunchKernelGGL((issue_mix_kernel<16, 40, 16, 8, 16>), g, t, 0, st, out, iters, 0.f); break;
    case 4: hipLaunchKernelGGL((issue_mix_kernel<0, 40, 16, 0, 0>), g, t, 0, st, out, iters, 0.f); break;
    default: hipLaunchKernelGGL((issue_mix_kernel<0, 0, 0, 8, 16>), g, t, 0, st, out, iters, 0.f); break;
  }
  return hipGetLastError() == hipSuccess ? 0 : -6;
}
