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
//
// Rows of whole scale groups (k a multiple of the group, the usual case) take a faster form of the same
// order, lane = weight row: a wave takes 64 rows and ONE segment index, i.e. the same columns of every row,
// so an activation is one broadcast read for all lanes and the lanes never diverge; it folds the (up to
// three) planes of its segment side by side, one accumulator per plane and token, and writes the scaled
// terms to a workspace; a second kernel adds the terms of an output in the pinned order. (rows x segments
// waves instead of rows workgroups of which half the lanes idle: 4096 x 4096, two planes: 210 -> about 20 us
// for one token.)
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

// trits local .. local+15 of a plane (local a multiple of 16; all 16 lie inside the plane)
__device__ __forceinline__ void trits16(const uint8_t *p, unsigned nbytes, unsigned local, unsigned codec, int (&tr)[16]) {
  if (codec == TK_SALT_V2_D2) {
    const uint8_t *q = p + (local >> 2);
    const unsigned w = (unsigned)gload(q) | ((unsigned)gload(q + 1) << 8) | ((unsigned)gload(q + 2) << 16) | ((unsigned)gload(q + 3) << 24);
#pragma unroll
    for (int u = 0; u < 16; ++u) tr[u] = (int)((w >> (2 * u)) & 3u) - 1;
    return;
  }
  if (codec == TK_SALT_V2_B3) {
    // five bytes hold 25 digits from trit b0 * 5 on: all of them as 2-bit fields of one 64-bit word, shifted
    // to the first trit wanted (a byte is below 243, so (b * 171) >> 9 is b / 3 exactly)
    const unsigned b0 = local / 5u, r = local - b0 * 5u;
    unsigned long long fields = 0;
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      const unsigned b = gload(p + min(b0 + (unsigned)i, nbytes - 1u));
      const unsigned q1 = (b * 171u) >> 9, q2 = (q1 * 171u) >> 9, q3 = (q2 * 171u) >> 9, q4 = (q3 * 171u) >> 9;
      const unsigned d = (b - 3u * q1) | ((q1 - 3u * q2) << 2) | ((q2 - 3u * q3) << 4) | ((q3 - 3u * q4) << 6) | (q4 << 8);
      fields |= (unsigned long long)d << (10 * i);
    }
    fields >>= 2u * r;
#pragma unroll
    for (int u = 0; u < 16; ++u) tr[u] = (int)((unsigned)(fields >> (2 * u)) & 3u) - 1;
    return;
  }
  // S34: four groups of five bits from bit (local / 4) * 5 on (local is a multiple of 16: the offset inside the
  // first byte is 0 or 4, so four bytes hold the twenty bits)
  const unsigned bit = (local >> 2) * 5u, byte = bit >> 3;
  unsigned word = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) word |= (unsigned)gload(p + min(byte + (unsigned)i, nbytes - 1u)) << (8 * i);
  word >>= bit & 7u;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const unsigned code = (word >> (5 * g)) & 31u, zero = code & 3u;
#pragma unroll
    for (int slot = 0; slot < 4; ++slot) {
      const unsigned sign = (unsigned)slot - ((unsigned)slot > zero ? 1u : 0u);
      const int v = (code >> (2u + sign)) & 1u ? 1 : -1;
      tr[g * 4 + slot] = (unsigned)slot == zero ? 0 : v;
    }
  }
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

// ---- lane = row (k % group == 0) ----
// terms[(tok * nseg * 3 + s * 3 + j) * n + row]: the product of plane j of segment s of `row` for token `tok`
// (planes a tile does not have are left unwritten and never read).
template <int MT>
__global__ __launch_bounds__(64) void tk_salt_v2_terms_kernel(TkSaltV2 t, const float *__restrict__ act, unsigned tok_begin,
                                                              unsigned tok_end, float *__restrict__ terms,
                                                              unsigned *__restrict__ flag) {
  const unsigned lane = threadIdx.x, row = blockIdx.x * 64u + lane, s = blockIdx.y;
  const unsigned tok0 = tok_begin + blockIdx.z * MT;
  const unsigned mt = min((unsigned)MT, tok_end - tok0);
  const bool active = row < t.n;
  const unsigned rowc = active ? row : t.n - 1u;
  const unsigned nseg = t.k / t.group, c0 = s * t.group;
  const unsigned long long lo = (unsigned long long)rowc * t.k + c0;
  const unsigned tile = (unsigned)(lo >> 8), local0 = (unsigned)(lo & 255ull);
  const TileView tv = tile_view(t, tile);
  const unsigned full_bytes = plane_bytes(t.codec, 256u), cur_bytes = plane_bytes(t.codec, tv.len);
  const unsigned full_groups = 256u / t.group, cur_groups = (tv.len + t.group - 1u) / t.group;
  const unsigned codec = t.codec, group = t.group;
  const uint8_t *pj[3];
#pragma unroll
  for (int j = 0; j < 3; ++j)  // (a plane the tile does not have reads the last one it has; its sums are dropped)
    pj[j] = t.payload + (size_t)tv.begin * full_bytes + (size_t)min((unsigned)j, tv.planes - 1u) * cur_bytes;
  float acc[3][MT];
#pragma unroll
  for (int j = 0; j < 3; ++j)
#pragma unroll
    for (int x = 0; x < MT; ++x) acc[j][x] = 0.0f;
  // the segment's activations, [column][token], once per workgroup (every lane reads the same ones: LDS
  // broadcasts); the first row block checks that they are finite
  __shared__ float sh_act[128 * MT];
  bool bad = false;
  const bool checks = blockIdx.x == 0;
  for (unsigned e = lane; e < group * MT; e += 64u) {
    const unsigned col = e / MT, x = e % MT;  // (MT is a power of two)
    const float v = x < mt ? gload(act + (size_t)(tok0 + x) * t.k + c0 + col) : 0.0f;
    if (checks) bad |= !(fabsf(v) <= 3.402823466e38f);
    sh_act[e] = v;
  }
  __syncthreads();
  // sixteen columns at a time: their codes are requested together (the loads do not depend on the sums), then
  // folded in column order
  for (unsigned o0 = 0; o0 < group; o0 += 16) {
    int tr[3][16];
#pragma unroll
    for (int j = 0; j < 3; ++j) trits16(pj[j], cur_bytes, local0 + o0, codec, tr[j]);
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      float a[MT];
#pragma unroll
      for (int x = 0; x < MT; ++x) a[x] = sh_act[(o0 + u) * MT + x];
#pragma unroll
      for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int x = 0; x < MT; ++x) {
          const float up = __fadd_rn(acc[j][x], a[x]), down = __fsub_rn(acc[j][x], a[x]);
          acc[j][x] = tr[j][u] > 0 ? up : (tr[j][u] < 0 ? down : acc[j][x]);  // a zero trit skips the activation
        }
    }
  }
  if (active) {
    const unsigned gidx = local0 / group;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      if ((unsigned)j >= tv.planes) continue;
      const float sc = f16_to_f32(gload(t.scales + (size_t)tv.begin * full_groups + (size_t)j * cur_groups + gidx));
#pragma unroll
      for (int x = 0; x < MT; ++x)
        if ((unsigned)x < mt)
          terms[((size_t)(tok0 + x - tok_begin) * nseg * 3u + (size_t)s * 3u + j) * t.n + row] = __fmul_rn(acc[j][x], sc);
    }
  }
  if (bad) atomicOr(flag, 1u);
}

// out[tok, row] = the terms of the row's segments added in the pinned order: segments ascending, planes ascending
__global__ __launch_bounds__(TK_WG) void tk_salt_v2_sum_kernel(TkSaltV2 t, const float *__restrict__ terms, unsigned tok_begin,
                                                               unsigned tok_end, float *__restrict__ out,
                                                               unsigned *__restrict__ flag) {
  const size_t idx = (size_t)blockIdx.x * TK_WG + threadIdx.x;
  if (idx >= (size_t)(tok_end - tok_begin) * t.n) return;
  const unsigned tl = (unsigned)(idx / t.n), row = (unsigned)(idx - (size_t)tl * t.n);
  const unsigned nseg = t.k / t.group;
  float accumulator = 0.0f;
  // sixteen segments at a time: plane counts and terms are requested together, then added in order (a plane
  // the tile does not have is not read and not added)
  for (unsigned s0 = 0; s0 < nseg; s0 += 16) {
    unsigned planes[16];
    float term[16][3];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const unsigned s = min(s0 + u, nseg - 1u);
      const unsigned tile = (unsigned)(((unsigned long long)row * t.k + (unsigned long long)s * t.group) >> 8);
      planes[u] = s0 + u < nseg ? gload(t.tile_begin + tile + 1) - gload(t.tile_begin + tile) : 0u;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u)
#pragma unroll
      for (int j = 0; j < 3; ++j)
        term[u][j] = (unsigned)j < planes[u] ? gload(terms + ((size_t)tl * nseg * 3u + (size_t)(s0 + u) * 3u + j) * t.n + row) : 0.0f;
#pragma unroll
    for (int u = 0; u < 16; ++u)
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const float next = __fadd_rn(accumulator, term[u][j]);
        accumulator = (unsigned)j < planes[u] ? next : accumulator;
      }
  }
  // an accumulator that left the finite range never comes back (inf - inf is NaN): the end result tells
  if (!(fabsf(accumulator) <= 3.402823466e38f)) atomicOr(flag, 1u);
  out[(size_t)(tok_begin + tl) * t.n + row] = accumulator;
}

// The results leave the staging buffer only when no activation and no result was found non-finite.
__global__ __launch_bounds__(TK_WG) void tk_salt_v2_commit_kernel(const float *__restrict__ tmp, float *__restrict__ out, size_t count,
                                                                  const unsigned *__restrict__ flag) {
  if (gload(flag)) return;
  const size_t idx = (size_t)blockIdx.x * TK_WG + threadIdx.x;
  if (idx < count) out[idx] = gload(tmp + idx);
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

// floats of workspace per token the lane = row form needs (0: the matrix does not take that form)
size_t tk_salt_v2_term_floats(const TkSaltV2 &t) {
  if (!t.group || t.k % t.group != 0 || t.k / t.group > 65535u) return 0;
  return (size_t)(t.k / t.group) * 3 * t.n;
}

// terms: workspace of term_tokens * tk_salt_v2_term_floats(t) floats (term_tokens >= 1), or null for the form
// that needs none
hipError_t tk_launch_salt_v2_forward(hipStream_t s, const TkSaltV2 &t, const float *act, size_t m, float *tmp, unsigned *flag,
                                     float *terms, size_t term_tokens) {
  if (!m || !t.n) return hipSuccess;
  if (terms && term_tokens && tk_salt_v2_term_floats(t)) {
    const unsigned nseg = t.k / t.group;
    for (size_t b = 0; b < m; b += term_tokens) {
      const unsigned e = (unsigned)(b + term_tokens < m ? b + term_tokens : m), cnt = e - (unsigned)b;
      const dim3 block(64);
      if (cnt == 1) {
        hipLaunchKernelGGL(tk_salt_v2_terms_kernel<1>, dim3((t.n + 63) / 64, nseg, cnt), block, 0, s, t, act, (unsigned)b, e, terms, flag);
      } else if (cnt <= 4) {
        hipLaunchKernelGGL(tk_salt_v2_terms_kernel<4>, dim3((t.n + 63) / 64, nseg, 1), block, 0, s, t, act, (unsigned)b, e, terms, flag);
      } else {
        hipLaunchKernelGGL(tk_salt_v2_terms_kernel<8>, dim3((t.n + 63) / 64, nseg, (cnt + 7) / 8), block, 0, s, t, act, (unsigned)b, e, terms, flag);
      }
      hipError_t err = hipGetLastError();
      if (err != hipSuccess) return err;
      const size_t outs = (size_t)cnt * t.n;
      hipLaunchKernelGGL(tk_salt_v2_sum_kernel, dim3((unsigned)((outs + TK_WG - 1) / TK_WG)), dim3(TK_WG), 0, s, t, terms, (unsigned)b, e, tmp, flag);
      err = hipGetLastError();
      if (err != hipSuccess) return err;
    }
    return hipSuccess;
  }
  const size_t lds = tk_salt_v2_lds_bytes(t.k, t.group);
  if (lds > 64 * 1024) {
    hipError_t e = tk_raise_lds_limit((const void *)tk_salt_v2_forward_kernel, 160 * 1024);
    if (e != hipSuccess) return e;
  }
  const dim3 grid(t.n, (unsigned)((m + TK_SALT_V2_TOKENS - 1) / TK_SALT_V2_TOKENS));
  hipLaunchKernelGGL(tk_salt_v2_forward_kernel, grid, dim3(64), lds, s, t, act, (unsigned)m, tmp, flag);
  return hipGetLastError();
}

hipError_t tk_launch_salt_v2_commit(hipStream_t s, const float *tmp, float *out, size_t count, const unsigned *flag) {
  if (!count) return hipSuccess;
  hipLaunchKernelGGL(tk_salt_v2_commit_kernel, dim3((unsigned)((count + TK_WG - 1) / TK_WG)), dim3(TK_WG), 0, s, tmp, out, count, flag);
  return hipGetLastError();
}

hipError_t tk_launch_salt_v2_gather(hipStream_t s, const TkSaltV2 &t, const uint32_t *rows, size_t count, float *out) {
  const size_t total = count * t.k;
  if (!total) return hipSuccess;
  hipLaunchKernelGGL(tk_salt_v2_gather_kernel, dim3((unsigned)((total + TK_WG - 1) / TK_WG)), dim3(TK_WG), 0, s, t, rows, count, out);
  return hipGetLastError();
}
