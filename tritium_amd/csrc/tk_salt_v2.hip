// SALT V2 on gfx950: the exact forward and the row gather over resident codec payloads.
//
// The reference pins one scalar order per output (crates/tritium-cpu/src/salt_v2.rs:10-23): segments --
// the pieces of a weight row that lie in one 256-coefficient allocation tile and one scale group -- in
// ascending order; within a segment the tile's planes ascending; within a plane one f32 accumulator over
// the columns (add, subtract or skip by the trit), one multiply by the plane's f16 scale, one add into the
// output. Its own device kernel walks all of that with one thread per output
// (crates/tritium-cuda/kernels/salt_v2.cu:133-214). Here the terms of different segments, which do not
// depend on each other, are computed by different lanes: a workgroup takes one weight row and up to eight
// tokens, every lane folds whole segments (decoding each trit once for all tokens) and leaves the products
// in LDS; then one lane per token adds them in the pinned order. Same operations, same order per output,
// so the bits are those of the CPU reference.
//
// Compiled with -ffp-contract=off; the sums use explicit round-to-nearest adds and multiplies.

#include "tk_device.h"

namespace {

// bytes of one plane of `len` coefficients (crates/tritium-format/src/salt_v2.rs:160-258)
__device__ __forceinline__ unsigned plane_bytes(unsigned codec, unsigned len) {
  if (codec == TK_SALT_V2_D2) return (len + 3u) / 4u;
  if (codec == TK_SALT_V2_B3) return (len + 4u) / 5u;
  return ((len + 3u) / 4u * 5u + 7u) / 8u;
}

// trit `local` of a plane whose payload starts at p (salt_v2.rs:289-322,358-392,454-481)
__device__ __forceinline__ int trit_at(const uint8_t *p, unsigned nbytes, unsigned local, unsigned codec) {
  if (codec == TK_SALT_V2_D2) return (int)((gload(p + (local >> 2)) >> ((local & 3u) * 2u)) & 3u) - 1;
  if (codec == TK_SALT_V2_B3) {
    const unsigned place[5] = {1u, 3u, 9u, 27u, 81u};
    return (int)((gload(p + local / 5u) / place[local % 5u]) % 3u) - 1;
  }
  const unsigned bit = (local >> 2) * 5u, byte = bit >> 3;
  unsigned word = gload(p + byte);
  if (byte + 1u < nbytes) word |= (unsigned)gload(p + byte + 1u) << 8;
  const unsigned code = (word >> (bit & 7u)) & 31u, slot = local & 3u, zero = code & 3u;
  if (slot == zero) return 0;
  const unsigned sign = slot - (slot > zero ? 1u : 0u);
  return (code >> (2u + sign)) & 1u ? 1 : -1;
}

struct TileView {
  unsigned begin, planes, len;
};
__device__ __forceinline__ TileView tile_view(const TkSaltV2 &t, unsigned tile) {
  TileView v;
  v.begin = gload(t.tile_begin + tile);
  v.planes = gload(t.tile_begin + tile + 1) - v.begin;
  const unsigned long long base = (unsigned long long)tile * 256ull;
  v.len = (unsigned)(t.total - base < 256ull ? t.total - base : 256ull);
  return v;
}

__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  _Float16 x;
  __builtin_memcpy(&x, &h, 2);
  return (float)x;  // exact
}

}  // namespace

// LDS: float term[segments][3 planes][tokens], then one plane count per segment.
// Segment boundaries are the multiples of the scale group (which divides the 256 of a tile).
__global__ __launch_bounds__(64) void tk_salt_v2_forward_kernel(TkSaltV2 t, const float *__restrict__ act, unsigned m,
                                                                float *__restrict__ out, unsigned *__restrict__ flag) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int MT = TK_SALT_V2_TOKENS;
  const unsigned row = blockIdx.x, tok0 = blockIdx.y * MT;
  const unsigned mt = min((unsigned)MT, m - tok0);
  const unsigned long long row_base = (unsigned long long)row * t.k, row_end = row_base + t.k;
  const unsigned long long first = row_base / t.group;
  const unsigned nseg = (unsigned)((row_end + t.group - 1) / t.group - first);
  float *term = (float *)smem;
  uint8_t *seg_planes = smem + (size_t)nseg * 3 * MT * sizeof(float);
  bool bad = false;

  for (unsigned s = threadIdx.x; s < nseg; s += blockDim.x) {
    const unsigned long long lo = max(row_base, (first + s) * t.group), hi = min(row_end, (first + s + 1) * t.group);
    const unsigned tile = (unsigned)(lo >> 8), local = (unsigned)(lo & 255ull), seg = (unsigned)(hi - lo);
    const TileView tv = tile_view(t, tile);
    const unsigned group = local / t.group;
    const unsigned full_bytes = plane_bytes(t.codec, 256u), cur_bytes = plane_bytes(t.codec, tv.len);
    const unsigned full_groups = 256u / t.group, cur_groups = (tv.len + t.group - 1u) / t.group;
    const unsigned col0 = (unsigned)(lo - row_base);
    seg_planes[s] = (uint8_t)tv.planes;
    for (unsigned j = 0; j < tv.planes; ++j) {
      const uint8_t *p = t.payload + (size_t)tv.begin * full_bytes + (size_t)j * cur_bytes;
      float acc[MT];
#pragma unroll
      for (int x = 0; x < MT; ++x) acc[x] = 0.0f;
      for (unsigned o = 0; o < seg; ++o) {
        const int tr = trit_at(p, cur_bytes, local + o, t.codec);
        if (j == 0) {  // every activation of these tokens passes here once per row: the finiteness check
#pragma unroll
          for (int x = 0; x < MT; ++x)
            if ((unsigned)x < mt) bad |= !(fabsf(gload(act + (size_t)(tok0 + x) * t.k + col0 + o)) <= 3.402823466e38f);
        }
        if (tr == 0) continue;
#pragma unroll
        for (int x = 0; x < MT; ++x) {
          if ((unsigned)x >= mt) continue;
          const float a = gload(act + (size_t)(tok0 + x) * t.k + col0 + o);
          acc[x] = tr > 0 ? __fadd_rn(acc[x], a) : __fsub_rn(acc[x], a);
        }
      }
      const float sc = f16_to_f32(gload(t.scales + (size_t)tv.begin * full_groups + (size_t)j * cur_groups + group));
#pragma unroll
      for (int x = 0; x < MT; ++x) term[((size_t)s * 3 + j) * MT + x] = __fmul_rn(acc[x], sc);
    }
  }
  __syncthreads();
  if (threadIdx.x < mt) {
    float accumulator = 0.0f;
    for (unsigned s = 0; s < nseg; ++s)
      for (unsigned j = 0; j < seg_planes[s]; ++j) accumulator = __fadd_rn(accumulator, term[((size_t)s * 3 + j) * MT + threadIdx.x]);
    // an accumulator that left the finite range never comes back (inf - inf is NaN): the end result tells
    bad |= !(fabsf(accumulator) <= 3.402823466e38f);
    out[(size_t)(tok0 + threadIdx.x) * t.n + row] = accumulator;
  }
  if (bad) atomicOr(flag, 1u);
}

// One thread per gathered coefficient (crates/tritium-cuda/kernels/salt_v2.cu:218-304).
__global__ __launch_bounds__(TK_WG) void tk_salt_v2_gather_kernel(TkSaltV2 t, const uint32_t *__restrict__ rows, size_t count,
                                                                  float *__restrict__ out) {
  const size_t idx = (size_t)blockIdx.x * TK_WG + threadIdx.x;
  if (idx >= count * t.k) return;
  const size_t sel = idx / t.k;
  const unsigned col = (unsigned)(idx - sel * t.k);
  const unsigned long long c = (unsigned long long)gload(rows + sel) * t.k + col;
  const unsigned tile = (unsigned)(c >> 8), local = (unsigned)(c & 255ull);
  const TileView tv = tile_view(t, tile);
  const unsigned full_bytes = plane_bytes(t.codec, 256u), cur_bytes = plane_bytes(t.codec, tv.len);
  const unsigned full_groups = 256u / t.group, cur_groups = (tv.len + t.group - 1u) / t.group, group = local / t.group;
  float acc = 0.0f;
  for (unsigned j = 0; j < tv.planes; ++j) {
    const int tr = trit_at(t.payload + (size_t)tv.begin * full_bytes + (size_t)j * cur_bytes, cur_bytes, local, t.codec);
    const float sc = f16_to_f32(gload(t.scales + (size_t)tv.begin * full_groups + (size_t)j * cur_groups + group));
    if (tr > 0) acc = __fadd_rn(acc, sc);
    else if (tr < 0) acc = __fsub_rn(acc, sc);
  }
  out[idx] = acc;
}

size_t tk_salt_v2_lds_bytes(size_t k, size_t group) {
  const size_t nseg = k / group + 2;  // a row that starts and ends inside a group touches two more
  return nseg * 3 * TK_SALT_V2_TOKENS * sizeof(float) + ((nseg + 15) & ~(size_t)15);
}

hipError_t tk_launch_salt_v2_forward(hipStream_t s, const TkSaltV2 &t, const float *act, size_t m, float *tmp, unsigned *flag) {
  if (!m || !t.n) return hipSuccess;
  const size_t lds = tk_salt_v2_lds_bytes(t.k, t.group);
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void *)tk_salt_v2_forward_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
  }
  const dim3 grid(t.n, (unsigned)((m + TK_SALT_V2_TOKENS - 1) / TK_SALT_V2_TOKENS));
  hipLaunchKernelGGL(tk_salt_v2_forward_kernel, grid, dim3(64), lds, s, t, act, (unsigned)m, tmp, flag);
  return hipGetLastError();
}

hipError_t tk_launch_salt_v2_gather(hipStream_t s, const TkSaltV2 &t, const uint32_t *rows, size_t count, float *out) {
  const size_t total = count * t.k;
  if (!total) return hipSuccess;
  hipLaunchKernelGGL(tk_salt_v2_gather_kernel, dim3((unsigned)((total + TK_WG - 1) / TK_WG)), dim3(TK_WG), 0, s, t, rows, count, out);
  return hipGetLastError();
}
