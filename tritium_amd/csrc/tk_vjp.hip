// TernaryBackend::mpgemm_projected_vjp on the device (crates/tritium-spec/src/lib.rs:93-117, 217-232):
// the three gradients of one packed ternary mpGEMM, each output element summed by one thread in the
// index order and with the unfused f32 operations of the CPU backend's scalar path
// (crates/tritium-cpu/src/kernel.rs:150-189, 281-317), so the results carry its bits.
//
//   grad_act[m,k] = sum_n upstream[m,n] * (trit[n,k] * scales[n])     n = 0, 1, ...
//   grad_w[n,k]   = sum_m upstream[m,n] * act[m,k]                    m = 0, 1, ...
//   grad_bias[n]  = sum_m upstream[m,n]                               m = 0, 1, ...
//
// Both matrix kernels are fp32 vector-ALU bound (one multiply and one add per term, kept apart for
// the rounding). Weights are read in the device layout of the forward kernels: the 1-KiB chunk of
// row tile t and K block kb holds, for lane group g = 0..3 and row r = 0..15, the 16 code bytes
// g*16 .. g*16+15 of that row's block at offset g*256 + r*16; byte i of a block holds the elements
// (i/32)*128 + s*32 + i%32 at bit pairs s = 0..3, code = trit + 1.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tk_internal.h"

#define TKV_GLOBAL __attribute__((address_space(1)))
#ifndef TKV_ACT_TOK
#define TKV_ACT_TOK 4  // tokens per thread of the grad_act kernel (2: 3.2 ms, 4: 2.9 ms, 8: 4.5 ms at M=2048 K=2560 N=6912)
#endif

namespace {

__device__ __forceinline__ float ldg(const float *p) { return *(const TKV_GLOBAL float *)p; }

// grad_act. A workgroup owns 4*TOK tokens x 4 K blocks; a thread owns TOK tokens x the 16 elements of
// one code dword (piece g, dword j of its K block), the four waves are the four token groups. Per tile
// of 16 weight rows the upstream values and scales pass through LDS (two buffers, one barrier a tile).
template <int TOK>
__global__ __launch_bounds__(256) void tk_vjp_act_kernel(const uint8_t *__restrict__ codes, int nb, int n, int k, int m,
                                                         const float *__restrict__ scales,
                                                         const float *__restrict__ grad_output,
                                                         float *__restrict__ grad_act) {
  constexpr int WT = 4 * TOK;            // tokens per workgroup
  __shared__ float s_up[2][WT][16];      // [buffer][token][row of the tile]
  __shared__ float s_sc[2][16];
  const int tid = threadIdx.x;
  const int set = tid >> 4, ls = tid & 15, g = ls >> 2, j = ls & 3;
  const int kb = blockIdx.x * 4 + (set & 3), mg = set >> 2;
  const int m0 = blockIdx.y * WT;
  const int kbc = min(kb, nb - 1);  // blocks past the end re-read the last one; nothing of them is stored
  const int n_tiles = (n + 15) >> 4;
  float acc[TOK][16];
#pragma unroll
  for (int i = 0; i < TOK; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;

  auto stage = [&](int buf, int t) {
    if (tid < WT * 16) {
      const int mi = m0 + (tid >> 4), ni = t * 16 + (tid & 15);
      s_up[buf][tid >> 4][tid & 15] = (mi < m && ni < n) ? ldg(grad_output + (size_t)mi * n + ni) : 0.0f;
    }
    if (tid < 16) s_sc[buf][tid] = (t * 16 + tid < n) ? ldg(scales + t * 16 + tid) : 0.0f;
  };
  stage(0, 0);
  __syncthreads();
  for (int t = 0; t < n_tiles; ++t) {
    const int buf = t & 1;
    if (t + 1 < n_tiles) stage(buf ^ 1, t + 1);
    const int rmax = min(16, n - t * 16);
    const uint8_t *cp = codes + ((size_t)t * nb + kbc) * 1024 + g * 256 + j * 4;
    uint32_t w[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) w[r] = *(const TKV_GLOBAL uint32_t *)(cp + r * 16);  // padding rows of the last tile exist
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (r < rmax) {  // uniform
        const float s = s_sc[buf][r];
        float u[TOK];
#pragma unroll
        for (int i = 0; i < TOK; ++i) u[i] = s_up[buf][mg * TOK + i][r];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          // e = b*4 + sl: byte b of the dword, bit pair sl
          const int code = (int)((w[r] >> (8 * (e >> 2) + 2 * (e & 3))) & 3u);
          const float projected = __fmul_rn((float)(code - 1), s);
#pragma unroll
          for (int i = 0; i < TOK; ++i) acc[i][e] = __fadd_rn(acc[i][e], __fmul_rn(u[i], projected));
        }
      }
    }
    __syncthreads();
  }
  if (kb >= nb) return;
  // byte b of this dword is byte i = g*16 + j*4 + b of the block: elements (g/2)*128 + sl*32 + (g%2)*16 + j*4 + b
  const int e0 = kb * 256 + (g >> 1) * 128 + (g & 1) * 16 + j * 4;
#pragma unroll
  for (int i = 0; i < TOK; ++i) {
    const int mi = m0 + mg * TOK + i;
    if (mi >= m) continue;
    float *row = grad_act + (size_t)mi * k;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int kk = e0 + sl * 32 + b;
        if (kk < k) *(TKV_GLOBAL float *)(row + kk) = acc[i][b * 4 + sl];
      }
  }
}

// grad_w. A workgroup owns 64 weight rows x 64 columns, a thread 4 x 4 of them; tokens pass through
// LDS sixteen at a time (two buffers, one barrier per sixteen).
__global__ __launch_bounds__(256) void tk_vjp_weight_kernel(int n, int k, int m, const float *__restrict__ act,
                                                            const float *__restrict__ grad_output,
                                                            float *__restrict__ grad_w) {
  __shared__ __attribute__((aligned(16))) float s_act[2][16][64];
  __shared__ __attribute__((aligned(16))) float s_up[2][16][64];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int k0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  float acc[4][4];
#pragma unroll
  for (int y = 0; y < 4; ++y)
#pragma unroll
    for (int x = 0; x < 4; ++x) acc[y][x] = 0.0f;
  auto stage = [&](int buf, int mt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = tid + 256 * q, i = idx >> 6, c = idx & 63;
      const int mi = mt * 16 + i;
      s_act[buf][i][c] = (mi < m && k0 + c < k) ? ldg(act + (size_t)mi * k + k0 + c) : 0.0f;
      s_up[buf][i][c] = (mi < m && n0 + c < n) ? ldg(grad_output + (size_t)mi * n + n0 + c) : 0.0f;
    }
  };
  const int m_tiles = (m + 15) >> 4;
  stage(0, 0);
  __syncthreads();
  for (int mt = 0; mt < m_tiles; ++mt) {
    const int buf = mt & 1;
    if (mt + 1 < m_tiles) stage(buf ^ 1, mt + 1);
    const int imax = min(16, m - mt * 16);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (i < imax) {  // uniform
        const float4 a = *(const float4 *)&s_act[buf][i][tx * 4];
        const float4 u = *(const float4 *)&s_up[buf][i][ty * 4];
        const float av[4] = {a.x, a.y, a.z, a.w}, uv[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int y = 0; y < 4; ++y)
#pragma unroll
          for (int x = 0; x < 4; ++x) acc[y][x] = __fadd_rn(acc[y][x], __fmul_rn(uv[y], av[x]));
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int y = 0; y < 4; ++y) {
    const int ni = n0 + ty * 4 + y;
    if (ni >= n) continue;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int kk = k0 + tx * 4 + x;
      if (kk < k) *(TKV_GLOBAL float *)(grad_w + (size_t)ni * k + kk) = acc[y][x];
    }
  }
}

// grad_bias. One thread per column walks the tokens in order; a wave covers 64 adjacent columns, and
// 32 loads are in flight per thread (the additions stay in token order).
__global__ __launch_bounds__(64) void tk_vjp_bias_kernel(int n, int m, const float *__restrict__ grad_output,
                                                         float *__restrict__ grad_bias) {
  const int ni = blockIdx.x * 64 + threadIdx.x;
  if (ni >= n) return;
  float acc = 0.0f;
  int mi = 0;
  for (; mi + 32 <= m; mi += 32) {
    float v[32];
#pragma unroll
    for (int q = 0; q < 32; ++q) v[q] = ldg(grad_output + (size_t)(mi + q) * n + ni);
#pragma unroll
    for (int q = 0; q < 32; ++q) acc = __fadd_rn(acc, v[q]);
  }
  for (; mi < m; ++mi) acc = __fadd_rn(acc, ldg(grad_output + (size_t)mi * n + ni));
  *(TKV_GLOBAL float *)(grad_bias + ni) = acc;
}

}  // namespace

// m, n, k > 0 for the matrix kernels (the caller has zero-filled or skipped the degenerate shapes);
// grad_act / grad_w / grad_bias may each be null to skip that output.
hipError_t tk_launch_projected_vjp(hipStream_t s, const uint8_t *codes, size_t nb, size_t n, size_t k, size_t m,
                                   const float *scales, const float *act, const float *grad_output, float *grad_act,
                                   float *grad_w, float *grad_bias) {
  if (grad_act && m && n && k) {
    constexpr int TOK = TKV_ACT_TOK;
    dim3 grid((unsigned)((nb + 3) / 4), (unsigned)((m + 4 * TOK - 1) / (4 * TOK)));
    hipLaunchKernelGGL(tk_vjp_act_kernel<TOK>, grid, dim3(256), 0, s, codes, (int)nb, (int)n, (int)k, (int)m, scales,
                       grad_output, grad_act);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (grad_w && m && n && k) {
    dim3 grid((unsigned)((k + 63) / 64), (unsigned)((n + 63) / 64));
    hipLaunchKernelGGL(tk_vjp_weight_kernel, grid, dim3(256), 0, s, (int)n, (int)k, (int)m, act, grad_output, grad_w);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (grad_bias && n) {
    hipLaunchKernelGGL(tk_vjp_bias_kernel, dim3((unsigned)((n + 63) / 64)), dim3(64), 0, s, (int)n, (int)m,
                       grad_output, grad_bias);
    return hipGetLastError();
  }
  return hipSuccess;
}
