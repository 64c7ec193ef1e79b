// Machine ceilings of one MI355X, measured with small kernels of their own (not part of
// libtpuhip.so): the dependent-launch floor, copy / read / write bandwidth at the sizes the
// layers have, strided 16-byte stores against full-line stores, the int8 MFMA peak, LDS
// fragment-read bandwidth, MFMAs fed from LDS at several wave tiles, L2-resident global loads
// (into registers and straight into LDS) and the issue rate of the vector-ALU instructions the
// requantisation is made of.  The rooflines quoted for the library's kernels lean on these
// figures rather than on datasheet peaks alone.
//   python -m tpu_compiler_amd.build --microbench && ./tpu_compiler_amd/machine_ceilings.bin
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <string>
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); exit(1); } } while (0)

static hipEvent_t e0, e1;
template <typename F> float time_us(F f, int iters = 20, int warm = 3) {
  for (int i = 0; i < warm; ++i) f();
  CK(hipEventRecord(e0));
  for (int i = 0; i < iters; ++i) f();
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  return ms * 1000.f / iters;
}

__global__ void k_empty(int *p) { if (p == (int *)1) *p = 0; }

// ---- copy: 16 B per lane, grid-stride
__global__ __launch_bounds__(256) void k_copy(const v4i *__restrict__ src, v4i *__restrict__ dst, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}
// 4 loads in flight per lane
__global__ __launch_bounds__(256) void k_copy4(const v4i *__restrict__ src, v4i *__restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    v4i a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    dst[i] = a; dst[i + stride] = b; dst[i + 2 * stride] = c; dst[i + 3 * stride] = d;
  }
  for (; i < n16; i += stride) dst[i] = src[i];
}
// read-only (sum) and write-only
__global__ __launch_bounds__(256) void k_read(const v4i *__restrict__ src, int *out, size_t n16) {
  v4i s = {0, 0, 0, 0};
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) s += src[i];
  if (s[0] + s[1] + s[2] + s[3] == 0x12345678) out[0] = 1;
}
__global__ __launch_bounds__(256) void k_write(v4i *__restrict__ dst, size_t n16) {
  v4i s = {1, 2, 3, 4};
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = s;
}
// strided 16-byte stores: lane l writes 16 B at row (base + l) * rowbytes + chunk * 16 (the conv epilogue's pattern)
__global__ __launch_bounds__(256) void k_write_rows(v4i *__restrict__ dst, int rows, int chunks) {
  v4i s = {1, 2, 3, 4};
  const int nw = gridDim.x * 4, w = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  for (int r0 = w * 64; r0 < rows; r0 += nw * 64) {
    const int r = r0 + lane;
    if (r < rows)
      for (int c = 0; c < chunks; ++c) dst[(size_t)r * chunks + c] = s;
  }
}
// same bytes, but lanes cover consecutive 16-byte chunks (full lines)
__global__ __launch_bounds__(256) void k_write_lin(v4i *__restrict__ dst, int rows, int chunks) {
  v4i s = {1, 2, 3, 4};
  const int nw = gridDim.x * 4, w = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  const size_t per = (size_t)64 * chunks;   // chunks of 64 rows
  for (int r0 = w * 64; r0 < rows; r0 += nw * 64) {
    const size_t base = (size_t)r0 * chunks;
    const size_t lim = (size_t)rows * chunks;
    for (int c = 0; c < chunks; ++c) {
      const size_t i = base + (size_t)c * 64 + lane;
      if (i < lim && i < base + per) dst[i] = s;
    }
  }
}

// ---- MFMA peak
template <int WHICH>
__global__ __launch_bounds__(256) void k_mfma(int *out, int iters) {
  v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, 6, (int)threadIdx.x};
  if (WHICH == 0) {
    v16i c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; ++i) {
      c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
    }
    int s = 0;
    for (int k = 0; k < 16; ++k) s += c0[k] + c1[k] + c2[k] + c3[k];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  } else {
    v4i c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; ++i) {
      c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c3, 0, 0, 0);
    }
    int s = 0;
    for (int k = 0; k < 4; ++k) s += c0[k] + c1[k] + c2[k] + c3[k];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  }
}

// ---- LDS read bandwidth: every wave reads fragments (lane: row l&31, chunk (l>>5)) of swizzled 64-byte rows
template <int NT>
__global__ __launch_bounds__(NT) void k_ldsread(int *out, int iters) {
  __shared__ v4i lds[4096];   // 64 KB
  for (int i = threadIdx.x; i < 4096; i += NT) lds[i] = v4i{i, i, i, i};
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int frow = lane & 31, fk = lane >> 5;
  v4i s0 = {0, 0, 0, 0}, s1 = s0, s2 = s0, s3 = s0;
  int base = wave * 128;
  for (int i = 0; i < iters; ++i) {
    // four fragments of 32 rows x 32 bytes from a tile of 64-byte rows, chunk ^= (row >> 2) & 3
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int chunk = kk * 2 + fk;
      const int r0 = (base + frow) & 1023, r1 = (base + 32 + frow) & 1023;
      s0 += lds[r0 * 4 + (chunk ^ ((r0 >> 2) & 3))];
      s1 += lds[r1 * 4 + (chunk ^ ((r1 >> 2) & 3))];
      const int r2 = (base + 64 + frow) & 1023, r3 = (base + 96 + frow) & 1023;
      s2 += lds[r2 * 4 + (chunk ^ ((r2 >> 2) & 3))];
      s3 += lds[r3 * 4 + (chunk ^ ((r3 >> 2) & 3))];
    }
    base += 128;
  }
  v4i s = s0 + s1 + s2 + s3;
  out[blockIdx.x * NT + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}

// ---- MFMA fed from LDS: a wave owns TM x TN blocks; per 32-byte K slice it reads TM + TN fragments
template <int TM, int TN, int NT>
__global__ __launch_bounds__(NT) void k_mfma_lds(int *out, int iters) {
  __shared__ v4i lds[4096];
  for (int i = threadIdx.x; i < 4096; i += NT) lds[i] = v4i{i & 3, 1, i & 1, 2};
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int frow = lane & 31, fk = lane >> 5;
  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int k = 0; k < 16; ++k) acc[i][j][k] = 0;
  v4i fa[2][TM], fb[2][TN];
  int base = wave * 32;
  auto rd = [&](int fs, int kk) {
    const int chunk = kk * 2 + fk;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int r = (base + i * 32 + frow) & 511;
      fa[fs][i] = lds[r * 4 + (chunk ^ ((r >> 2) & 3))];
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int r = 512 + ((base + j * 32 + frow) & 511);
      fb[fs][j] = lds[r * 4 + (chunk ^ ((r >> 2) & 3))];
    }
  };
  rd(0, 0);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      rd((kk + 1) & 1, (kk + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[kk & 1][i], fb[kk & 1][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    base += 32;
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int k = 0; k < 16; ++k) s += acc[i][j][k];
  out[blockIdx.x * NT + threadIdx.x] = s;
}

// ---- global -> register loads from an L2-resident buffer: every workgroup streams the same `span` bytes
template <int PATTERN>   // 0: 1 KiB contiguous per wave load; 1: 32 rows x 32 B (rows of 256 B)
__global__ __launch_bounds__(256) void k_gload(const v4i *__restrict__ src, int *out, int span16, int iters) {
  v4i s0 = {0, 0, 0, 0}, s1 = s0, s2 = s0, s3 = s0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int off = (blockIdx.x * 1031 + wave * 257) * 64;
  for (int i = 0; i < iters; ++i) {
    int idx[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int o = (off + u * 64 * (PATTERN ? 8 : 1)) % span16;
      if (PATTERN == 0) idx[u] = (o + lane) % span16;
      else idx[u] = (o + (lane & 31) * 16 + (lane >> 5)) % span16;
    }
    s0 += src[idx[0]]; s1 += src[idx[1]]; s2 += src[idx[2]]; s3 += src[idx[3]];
    off += 64 * 4 * (PATTERN ? 8 : 1);
  }
  v4i s = s0 + s1 + s2 + s3;
  if (s[0] + s[1] + s[2] + s[3] == 0x12345678) out[0] = 1;
}

// ---- global -> LDS direct loads (16 bytes per lane), same source pattern 0
__global__ __launch_bounds__(256) void k_gload_lds(const v4i *__restrict__ src, int *out, int span16, int iters) {
  __shared__ v4i lds[4 * 4 * 64];   // per wave 4 slots of 1 KiB
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int off = (blockIdx.x * 1031 + wave * 257) * 64;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int o = (off + u * 64) % span16;
      const int idx = (o + lane) % span16;
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)(src + idx),
                                       (void __attribute__((address_space(3))) *)(lds + (wave * 4 + u) * 64), 16, 0, 0);
    }
    off += 64 * 4;
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  v4i s = lds[threadIdx.x];
  if (s[0] + s[1] + s[2] + s[3] == 0x12345678) out[0] = 1;
}

// ---- VALU op rates: 8 independent chains per lane, the 8 instructions of a trip written as one
// block (the compiler puts a wait state between separate asm statements).  x: %0..%7, q (64-bit): %8..%15, m: %16
#define V8(F) F(0, 8) F(1, 9) F(2, 10) F(3, 11) F(4, 12) F(5, 13) F(6, 14) F(7, 15)
template <int OP>
__global__ __launch_bounds__(256) void k_valu(int *out, int iters, int seed) {
  int x[8];
  long long q[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) { x[u] = threadIdx.x * 7 + u + seed; q[u] = x[u]; }
  const int m = seed | 0x40000001;
#define OPERANDS                                                                                              \
  : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]), "+v"(q[0]), \
    "+v"(q[1]), "+v"(q[2]), "+v"(q[3]), "+v"(q[4]), "+v"(q[5]), "+v"(q[6]), "+v"(q[7])                          \
  : "v"(m)                                                                                                    \
  : "vcc"
  for (int i = 0; i < iters; ++i) {
#define A(N, Q) "v_add_u32 %" #N ", %" #N ", %16\n"
    if (OP == 0) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_and_b32 %" #N ", %" #N ", %16\n"
    if (OP == 1) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_lshrrev_b32 %" #N ", 3, %" #N "\n"
    if (OP == 2) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_ashrrev_i32 %" #N ", %16, %" #N "\n"
    if (OP == 3) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_mov_b32 %" #N ", %16\n"
    if (OP == 4) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_fma_f32 %" #N ", %" #N ", %16, %" #N "\n"
    if (OP == 5) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_lshlrev_b32 %" #N ", 3, %" #N "\n"
    if (OP == 6) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_max_i32 %" #N ", %" #N ", %16\n"
    if (OP == 7) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_med3_i32 %" #N ", %" #N ", %16, 64\n"
    if (OP == 8) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_add3_u32 %" #N ", %" #N ", %16, %16\n"
    if (OP == 9) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_perm_b32 %" #N ", %" #N ", %16, %16\n"
    if (OP == 10) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_alignbit_b32 %" #N ", %" #N ", %16, 31\n"
    if (OP == 11) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_cvt_pk_i16_i32 %" #N ", %" #N ", %16\n"
    if (OP == 12) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_pk_max_i16 %" #N ", %" #N ", %16\n"
    if (OP == 13) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_pk_mad_i16 %" #N ", %" #N ", %16, %" #N "\n"
    if (OP == 14) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_pk_ashrrev_i16 %" #N ", %16, %" #N "\n"
    if (OP == 15) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_mul_i32_i24 %" #N ", %" #N ", %16\n"
    if (OP == 16) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_mul_lo_u32 %" #N ", %" #N ", %16\n"
    if (OP == 17) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_mul_hi_i32 %" #N ", %" #N ", %16\n"
    if (OP == 18) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_dot4_i32_i8 %" #N ", %" #N ", %16, %" #N "\n"
    if (OP == 19) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_mad_i64_i32 %" #Q ", vcc, %" #N ", %16, %" #Q "\n"
    if (OP == 20) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_lshl_or_b32 %" #N ", %" #N ", 8, %16\n"
    if (OP == 21) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_sat_pk_u8_i16 %" #N ", %" #N "\n"
    if (OP == 22) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_fma_f64 %" #Q ", %" #Q ", %" #Q ", %" #Q "\n"
    if (OP == 23) asm volatile(V8(A) OPERANDS);
#undef A
#define A(N, Q) "v_cvt_i32_f64 %" #N ", %" #Q "\n"
    if (OP == 24) asm volatile(V8(A) OPERANDS);
#undef A
  }
#undef OPERANDS
  long long s = 0;
#pragma unroll
  for (int u = 0; u < 8; ++u) s += x[u] + q[u];
  out[blockIdx.x * 256 + threadIdx.x] = (int)s;
}
constexpr int kValuOps = 25;
const char *const kValuNames[kValuOps] = {
    "v_add_u32", "v_and_b32", "v_lshrrev_b32", "v_ashrrev_i32", "v_mov_b32", "v_fma_f32", "v_lshlrev_b32", "v_max_i32",
    "v_med3_i32", "v_add3_u32", "v_perm_b32", "v_alignbit_b32", "v_cvt_pk_i16_i32", "v_pk_max_i16", "v_pk_mad_i16",
    "v_pk_ashrrev_i16", "v_mul_i32_i24", "v_mul_lo_u32", "v_mul_hi_i32", "v_dot4_i32_i8", "v_mad_i64_i32",
    "v_lshl_or_b32", "v_sat_pk_u8_i16", "v_fma_f64", "v_cvt_i32_f64"};

int main(int argc, char **argv) {
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  hipDeviceProp_t prop; CK(hipGetDeviceProperties(&prop, 0));
  const int ncu = prop.multiProcessorCount;
  const double clk = prop.clockRate * 1e3;   // Hz
  printf("device %s CUs %d clock %.0f MHz LDS/block %zu\n", prop.name, ncu, clk / 1e6, prop.sharedMemPerBlock);
  int *out; CK(hipMalloc(&out, 64 << 20));
  const size_t big = 256u << 20;
  v4i *a, *b; CK(hipMalloc(&a, big)); CK(hipMalloc(&b, big));
  CK(hipMemset(a, 1, big)); CK(hipMemset(b, 2, big));

  printf("== launch floor\n");
  printf("empty kernel, back to back: %.2f us per launch\n", time_us([&] { hipLaunchKernelGGL(k_empty, dim3(1), dim3(64), 0, 0, out); }, 200));
  printf("empty kernel 1024 wgs:      %.2f us per launch\n", time_us([&] { hipLaunchKernelGGL(k_empty, dim3(1024), dim3(256), 0, 0, out); }, 200));

  printf("== copy (bytes = read + write), us and TB/s\n");
  for (double mb : {1.6, 3.2, 6.4, 12.8, 25.7, 51.4, 102.8}) {
    const size_t n16 = (size_t)(mb * 1e6 / 16);
    for (int wgs : {ncu * 2, ncu * 4, ncu * 8, 0}) {
      const int g = wgs ? wgs : (int)((n16 + 255) / 256);
      float t = time_us([&] { hipLaunchKernelGGL(k_copy, dim3(g), dim3(256), 0, 0, a, b, n16); });
      float t4 = time_us([&] { hipLaunchKernelGGL(k_copy4, dim3(g), dim3(256), 0, 0, a, b, n16); });
      printf("copy %6.1f MB grid %6d: %7.2f us %5.2f TB/s | 4-deep %7.2f us %5.2f TB/s\n", mb, g, t, 2 * mb / t, t4, 2 * mb / t4);
    }
    const int g = ncu * 8;
    float tr = time_us([&] { hipLaunchKernelGGL(k_read, dim3(g), dim3(256), 0, 0, a, out, n16); });
    float tw = time_us([&] { hipLaunchKernelGGL(k_write, dim3(g), dim3(256), 0, 0, b, n16); });
    printf("read %6.1f MB: %7.2f us %5.2f TB/s | write: %7.2f us %5.2f TB/s\n", mb, tr, mb / tr, tw, mb / tw);
  }
  printf("== strided 16-byte stores vs full-line stores, 25.7 MB\n");
  for (int chunks : {4, 16, 64}) {
    const int rows = (int)(25.7e6 / (chunks * 16));
    float t1 = time_us([&] { hipLaunchKernelGGL(k_write_rows, dim3(ncu * 8), dim3(256), 0, 0, b, rows, chunks); });
    float t2 = time_us([&] { hipLaunchKernelGGL(k_write_lin, dim3(ncu * 8), dim3(256), 0, 0, b, rows, chunks); });
    printf("row bytes %4d: lane-per-row %7.2f us %5.2f TB/s | linear %7.2f us %5.2f TB/s\n", chunks * 16, t1, 25.7 / t1, t2, 25.7 / t2);
  }

  printf("== MFMA peak\n");
  for (int wgs : {ncu, ncu * 2, ncu * 4}) {
    const int iters = 4000;
    float t0 = time_us([&] { hipLaunchKernelGGL(k_mfma<0>, dim3(wgs), dim3(256), 0, 0, out, iters); }, 5, 1);
    float t1 = time_us([&] { hipLaunchKernelGGL(k_mfma<1>, dim3(wgs), dim3(256), 0, 0, out, iters); }, 5, 1);
    const double n = (double)wgs * 4 * iters * 4;
    printf("wgs %5d: 32x32x32 %.0f TOP/s (%.1f clk per MFMA per SIMD at %.0f MHz) | 16x16x64 %.0f TOP/s\n", wgs,
           n * 65536 / t0 / 1e6, t0 * 1e-6 * clk / (n / (ncu * 4)), clk / 1e6, n * 32768 / t1 / 1e6);
  }

  printf("== LDS fragment reads (ds_read_b128), bytes per clock per CU at the nominal clock\n");
  {
    const int iters = 2000;
    float t4 = time_us([&] { hipLaunchKernelGGL(k_ldsread<256>, dim3(ncu), dim3(256), 0, 0, out, iters); }, 5, 1);
    float t8 = time_us([&] { hipLaunchKernelGGL(k_ldsread<512>, dim3(ncu), dim3(512), 0, 0, out, iters); }, 5, 1);
    float t16 = time_us([&] { hipLaunchKernelGGL(k_ldsread<1024>, dim3(ncu), dim3(1024), 0, 0, out, iters); }, 5, 1);
    auto bpc = [&](float t, int waves) { return (double)waves * iters * 8 * 1024 / (t * 1e-6 * clk); };
    printf("4 waves: %.1f B/clk/CU | 8 waves: %.1f | 16 waves: %.1f\n", bpc(t4, 4), bpc(t8, 8), bpc(t16, 16));
  }

  printf("== MFMA fed from LDS fragments (no global loads), 1 workgroup per CU unless noted\n");
  {
    const int iters = 2000;
#define RUN(TM, TN, NT, WGS)                                                                                   \
  {                                                                                                            \
    float t = time_us([&] { hipLaunchKernelGGL((k_mfma_lds<TM, TN, NT>), dim3(WGS), dim3(NT), 0, 0, out, iters); }, 5, 1); \
    const double n = (double)(WGS) * (NT / 64) * iters * 2 * TM * TN;                                          \
    printf("wave tile %dx%d, %d waves/wg, %d wgs: %.0f TOP/s\n", TM * 32, TN * 32, NT / 64, WGS, n * 65536 / t / 1e6); \
  }
    RUN(1, 1, 256, ncu) RUN(1, 2, 256, ncu) RUN(2, 2, 256, ncu) RUN(2, 4, 256, ncu) RUN(4, 4, 256, ncu)
    RUN(1, 2, 512, ncu) RUN(2, 2, 512, ncu) RUN(2, 4, 512, ncu)
    RUN(1, 2, 256, ncu * 2) RUN(2, 2, 256, ncu * 2) RUN(1, 2, 256, ncu * 3) RUN(2, 2, 256, ncu * 3)
#undef RUN
  }

  printf("== global loads of an L2-resident span by every workgroup (16 B per lane), B/clk/CU\n");
  for (int span_kb : {64, 1024, 16384}) {
    const int span16 = span_kb * 64, iters = 500;
    for (int wgs : {ncu, ncu * 2, ncu * 4}) {
      float t0 = time_us([&] { hipLaunchKernelGGL(k_gload<0>, dim3(wgs), dim3(256), 0, 0, a, out, span16, iters); }, 5, 1);
      float t1 = time_us([&] { hipLaunchKernelGGL(k_gload<1>, dim3(wgs), dim3(256), 0, 0, a, out, span16, iters); }, 5, 1);
      float t2 = time_us([&] { hipLaunchKernelGGL(k_gload_lds, dim3(wgs), dim3(256), 0, 0, a, out, span16, iters); }, 5, 1);
      const double bytes = (double)wgs * 4 * iters * 4 * 1024;
      printf("span %6d KB wgs %5d: contiguous %.1f | 32 rows x 32 B %.1f | direct to LDS %.1f  B/clk/CU (%.2f / %.2f / %.2f TB/s)\n", span_kb,
             wgs, bytes / (t0 * 1e-6 * clk) / ncu, bytes / (t1 * 1e-6 * clk) / ncu, bytes / (t2 * 1e-6 * clk) / ncu,
             bytes / t0 / 1e6, bytes / t1 / 1e6, bytes / t2 / 1e6);
    }
  }

  printf("== VALU: clocks per wave64 instruction per SIMD at 1, 2, 4 and 8 waves per SIMD (8 independent chains per wave)\n");
  {
    const int iters = 4000;
    const int wps[4] = {1, 2, 4, 8};
    static float t[4][kValuOps];
    for (int wi = 0; wi < 4; ++wi) {
      const int wgs = ncu * wps[wi];   // 4 waves per workgroup: one per SIMD
#define V(OP) t[wi][OP] = time_us([&] { hipLaunchKernelGGL(k_valu<OP>, dim3(wgs), dim3(256), 0, 0, out, iters, 3); }, 3, 1);
      V(0) V(1) V(2) V(3) V(4) V(5) V(6) V(7) V(8) V(9) V(10) V(11) V(12) V(13) V(14) V(15) V(16) V(17) V(18) V(19) V(20)
      V(21) V(22) V(23) V(24)
#undef V
    }
    for (int op = 0; op < kValuOps; ++op) {
      printf("%-18s", kValuNames[op]);
      for (int wi = 0; wi < 4; ++wi) printf(" %6.2f", t[wi][op] * 1e-6 * clk / ((double)wps[wi] * iters * 8));
      printf(" clk\n");
    }
  }
  CK(hipDeviceSynchronize());
  printf("done\n");
  return 0;
}
