// Device-side helpers shared by the kernel translation units: address-space-qualified loads and
// stores, the 2-bit code expansion, the reference-order fallback dot product, and the epilogues that
// turn int32 accumulators into outputs of the int8 and the float contract.
#pragma once

#include "tk_internal.h"

typedef int v4i __attribute__((ext_vector_type(4)));

#define TK_WG 256

// ------------------------------------------------------------------------------------------
// small helpers
// ------------------------------------------------------------------------------------------

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// float -> bf16, round to nearest even, NaN quieted with its sign and upper payload kept: gfx950's
// v_cvt_pk_bf16_f32 (what the vector conversion below compiles to) gives, for every one of the 2^32
// float bit patterns, the bits of the integer statement
//   nan ? (u >> 16) | 0x40 : (u + 0x7FFF + ((u >> 16) & 1)) >> 16
// (compared exhaustively on the device).
typedef float tk_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 tk_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
  const tk_f32x2 v = {lo, hi};
  const tk_bf16x2 h = __builtin_convertvector(v, tk_bf16x2);
  uint32_t bits;
  __builtin_memcpy(&bits, &h, 4);
  return bits;
}
__device__ __forceinline__ uint16_t f32_to_bf16_hw(float x) { return (uint16_t)f32x2_to_bf16x2(x, x); }
// The integer statement, for the decode kernels: their register budgets are fitted to it (the
// instruction form changed the allocation of two of them enough to spill).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Every pointer a kernel receives is device memory. Where the compiler cannot see that (a pointer
// read from a problem table), it would emit flat accesses, which also count on the LDS counter and
// serialise against LDS reads; these helpers state the address space.
#define TK_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ T gload(const T *p) {
  return *(const TK_GLOBAL T *)p;
}
template <typename T>
__device__ __forceinline__ void gstore(T *p, T v) {
  *(TK_GLOBAL T *)p = v;
}
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 gload16(const void *p) {
  const v4u v = *(const TK_GLOBAL v4u *)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}
// The same load for bytes that are read once per launch (the weight stream of the decode kernels): the non-temporal
// bit. A plain read probe on one MI355X streams 6.1-6.4 TB/s with ordinary 16-byte loads and 6.9-7.15 TB/s with the
// bit set, whatever the run length and the number of loads in flight (sc0 / sc1 alone change nothing).
#ifndef TK_STREAM_NT
#define TK_STREAM_NT 1
#endif
__device__ __forceinline__ uint4 gload16_stream(const void *p) {
#if TK_STREAM_NT
  const v4u v = __builtin_nontemporal_load((const TK_GLOBAL v4u *)p);
#else
  const v4u v = *(const TK_GLOBAL v4u *)p;
#endif
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float load_act(const void *p, int dtype, size_t idx) {
  return dtype == TK_BF16 ? bf16_to_f32(gload((const uint16_t *)p + idx)) : gload((const float *)p + idx);
}

__device__ __forceinline__ void store_out(void *out, int dtype, size_t idx, float v) {
  if (dtype == TK_BF16)
    gstore((uint16_t *)out + idx, f32_to_bf16_rne(v));
  else
    gstore((float *)out + idx, v);
}

// Fused residual add: out = residual + value, one f32 add (the epilogue of the reference's
// tq2_0_add_mpgemm_tiled_i8_scaled_residual, crates/tritium-cuda/kernels/tq2_0_add.cu:577-637).
// The residual has the layout and element type of the output; null = no residual.
__device__ __forceinline__ float with_residual(const void *residual, int dtype, size_t idx, float v) {
  if (!residual) return v;
  const float r = dtype == TK_BF16 ? bf16_to_f32(gload((const uint16_t *)residual + idx)) : gload((const float *)residual + idx);
  return __fadd_rn(r, v);
}

__device__ __forceinline__ v4i expand_codes(uint32_t w) {
  v4i b;
  b.x = (int)(w & 0x03030303u);
  b.y = (int)((w >> 2) & 0x03030303u);
  b.z = (int)((w >> 4) & 0x03030303u);
  b.w = (int)((w >> 6) & 0x03030303u);
  return b;
}

// 2-bit code (trit+1) of element k of row n from a T16 plane.
__device__ __forceinline__ int code_at(const uint8_t *codes, int nb, int n, int k) {
  int kb = k >> 8, e = k & 255;
  int c = e >> 7, s = (e & 127) >> 5, mm = e & 31;
  int byteidx = c * 32 + mm;
  int g = byteidx >> 4, bi = byteidx & 15;
  size_t off = (((size_t)(n >> 4) * nb + kb) * 64 + g * 16 + (n & 15)) * 16 + bi;
  return (codes[off] >> (2 * s)) & 3;
}

// The reference's contraction for one (token, output): one f32 accumulator, k in order,
// add / subtract / skip (crates/tritium-core/src/reference.rs:42-51). With a8 != 0 the activation
// is first quantized exactly as the host default does (crates/tritium-spec/src/lib.rs:369-374),
// kept in f32 so NaN survives. Takes plain scalars so callers keep their problem in registers.
__device__ __noinline__ float seq_dot_raw(const uint8_t *codes, int nb, int kdim, const void *raw_act,
                                          int raw_dtype, int n, int tok, int a8, float s, int gamma_zero) {
  float acc = 0.0f;
  for (int k = 0; k < kdim; ++k) {
    int code = code_at(codes, nb, n, k);
    if (code == 1) continue;
    float a = load_act(raw_act, raw_dtype, (size_t)tok * kdim + k);
    if (a8) {
      if (gamma_zero) {
        a = 0.0f;
      } else {
        a = rintf(__fmul_rn(a, s));
        a = a < -128.0f ? -128.0f : (a > 127.0f ? 127.0f : a);
      }
    }
    acc = (code == 2) ? __fadd_rn(acc, a) : __fsub_rn(acc, a);
  }
  return acc;
}

__device__ __forceinline__ float seq_dot(const TkProblem &pr, int p, int n, int tok, int a8) {
  const float s = a8 ? pr.aux[tok] : 0.0f;
  const int gamma_zero = a8 && pr.act_scale[tok] == 0.0f;
  return seq_dot_raw(pr.codes[p], pr.nb, pr.k, pr.raw_act, pr.raw_dtype, n, tok, a8, s, gamma_zero);
}

// Fold one plane's accumulators of one lane (4 consecutive operand rows starting at rowbase,
// output column n) into the running float outputs.
// The four digit rows of a token recombined: V = x3*2^24 + x2*2^16 + x1*2^8 + x0 (exact integers
// x_r = sum of trit*digit, |x_r| <= 128*K), scaled by the token's grid exponent. Three
// single-precision FMAs: the pairs (x3,x2) and (x1,x0) first, then their combination. The high pair
// is a multiple of 2^16 and the low pair is below 2^33, so whenever the two nearly cancel the high
// pair is small enough to be exact; otherwise the result has the magnitude of the high pair and each
// rounding is half an ulp of it: the value returned is within 1.5 ulp of the exact dot product (and
// equal to it when that is representable, e.g. for integer-valued activations), where a k-ordered
// f32 accumulation drifts by ~sqrt(K) ulp. Every kernel finishes through this one function, so
// their float results are bit-identical to each other. Double precision would round once, but runs
// at a fraction of the rate, and this sits on the decode path of every output.
__device__ __forceinline__ float digits_to_float(int x3, int x2, int x1, int x0, int exp) {
  const float hi = __builtin_fmaf((float)x3, 256.0f, (float)x2);
  const float lo = __builtin_fmaf((float)x1, 256.0f, (float)x0);
  return ldexpf(__builtin_fmaf(hi, 65536.0f, lo), exp);
}

__device__ __forceinline__ void fold_plane(const TkProblem &pr, int p, int n, int rowbase, v4i v,
                                           float out[4], bool first) {
  const float sc = pr.scales[p][n];
  if (pr.mode == TK_MODE_INT8) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      int m = rowbase + r;
      if (m < pr.R) {
        float f = __fmul_rn((float)(v[r] - pr.rowsum[m]), sc);
        out[r] = first ? f : __fadd_rn(out[r], f);
      }
    }
  } else {
    int tok = rowbase >> 2;
    if (tok < pr.M) {
      const int32_t *rs = pr.rowsum + rowbase;
      float val = digits_to_float(v[3] - rs[3], v[2] - rs[2], v[1] - rs[1], v[0] - rs[0], pr.exps[tok]);
      float f = __fmul_rn(val, sc);
      out[0] = first ? f : __fadd_rn(out[0], f);
    }
  }
}

__device__ __forceinline__ void finish_lane(const TkProblem &pr, int n, int rowbase, float out[4]) {
  if (pr.mode == TK_MODE_INT8) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      int m = rowbase + r;
      if (m >= pr.R) continue;
      float f = out[r];
      if (pr.flags && pr.flags[m]) {
        f = 0.0f;
        for (int p = 0; p < pr.planes; ++p) {
          float t = __fmul_rn(seq_dot(pr, p, n, m, 1), pr.scales[p][n]);
          f = p == 0 ? t : __fadd_rn(f, t);
        }
      }
      if (pr.act_scale) f = __fmul_rn(f, pr.act_scale[m]);
      store_out(pr.out, pr.out_dtype, (size_t)m * pr.n + n, with_residual(pr.residual, pr.out_dtype, (size_t)m * pr.n + n, f));
    }
  } else {
    int tok = rowbase >> 2;
    if (tok >= pr.M) return;
    float f = out[0];
    if (pr.flags && pr.flags[tok]) {
      f = 0.0f;
      for (int p = 0; p < pr.planes; ++p) {
        float t = __fmul_rn(seq_dot(pr, p, n, tok, 0), pr.scales[p][n]);
        f = p == 0 ? t : __fadd_rn(f, t);
      }
    }
    store_out(pr.out, pr.out_dtype, (size_t)tok * pr.n + n, with_residual(pr.residual, pr.out_dtype, (size_t)tok * pr.n + n, f));
  }
}

// raw int32 accumulators (single plane, INT8 mode): Σ_k q·trit
__device__ __forceinline__ void store_raw(const TkProblem &pr, int n, int rowbase, v4i v) {
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    int m = rowbase + r;
    if (m < pr.R) ((int32_t *)pr.out)[(size_t)m * pr.n + n] = v[r] - pr.rowsum[m];
  }
}

// The fields of a problem that the epilogues read, copied into registers once per kernel: read through
// a pointer into a problem table they would be fetched again after every store.
struct TkHot {
  void *out;
  const void *residual;
  const int32_t *rowsum;
  const float *act_scale;
  const int32_t *exps;
  const uint32_t *flags;
  int n, R, M, mode, out_dtype;
};
__device__ __forceinline__ TkHot make_hot(const TkProblem &pr) {
  TkHot h;
  h.out = pr.out;
  h.residual = pr.residual;
  h.rowsum = pr.rowsum;
  h.act_scale = pr.act_scale;
  h.exps = pr.exps;
  h.flags = pr.flags;
  h.n = pr.n;
  h.R = pr.R;
  h.M = pr.M;
  h.mode = pr.mode;
  h.out_dtype = pr.out_dtype;
  return h;
}

// The problem of a launch without a table is the first kernel argument. Read through an opaque
// pointer to the argument segment, its fields are fetched where they are used, as those of a table
// entry are; read as a by-value argument, the compiler loads all of them up front and keeps them in
// scalar registers for the whole kernel, which overflow into vector registers.
__device__ __forceinline__ const TkProblem *single_problem() {
  auto ka = __builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(ka));
  return (const TkProblem *)ka;
}

struct RowConst {
  int rs[4];       // row sums of the 4 operand rows this lane finishes
  float as[4];     // INT8: per-token activation scale (1.0 when absent)
  int exp;         // DIGITS: grid exponent of the token
  unsigned flag;   // any of the rows takes the exact fallback
};

// fallback flags of the 4 operand rows starting at rowbase (bit r = row r; DIGITS: bit 0 = the token)
__device__ __forceinline__ unsigned row_flags(const TkProblem &pr, int rowbase) {
  unsigned fl = 0;
  if (!pr.flags) return 0;
  if (pr.mode == TK_MODE_INT8) {
    for (int r = 0; r < 4; ++r)
      if (rowbase + r < pr.R && gload(pr.flags + rowbase + r)) fl |= 1u << r;
  } else {
    const int tok = rowbase >> 2;
    if (tok < pr.M && gload(pr.flags + tok)) fl = 1u;
  }
  return fl;
}

template <typename PR>
__device__ __forceinline__ RowConst load_row_const(const PR &pr, int rowbase) {
  RowConst rc;
  rc.exp = 0;
  rc.flag = 0;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = rowbase + r;
    rc.rs[r] = m < pr.R ? gload(pr.rowsum + m) : 0;
    rc.as[r] = 1.0f;
  }
  if (pr.mode == TK_MODE_INT8) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = rowbase + r;
      if (m < pr.R) {
        if (pr.act_scale) rc.as[r] = gload(pr.act_scale + m);
        if (pr.flags && gload(pr.flags + m)) rc.flag |= 1u << r;
      }
    }
  } else {
    const int tok = rowbase >> 2;
    if (tok < pr.M) {
      rc.exp = gload(pr.exps + tok);
      if (pr.flags && gload(pr.flags + tok)) rc.flag = 1u;
    }
  }
  return rc;
}

// One finished output of the int8 contract from the accumulator registers r of every plane.
template <int P>
__device__ __forceinline__ float int8_value(const v4i (&acc)[P], int r, const float (&sc)[P], const RowConst &rc,
                                            bool has_act_scale) {
  float f = 0.0f;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    float t = __fmul_rn((float)(acc[p][r] - rc.rs[r]), sc[p]);
    f = p == 0 ? t : __fadd_rn(f, t);
  }
  if (has_act_scale) f = __fmul_rn(f, rc.as[r]);
  return f;
}

// One finished output of the float contract from the accumulator registers of every plane.
template <int P>
__device__ __forceinline__ float digits_value(const v4i (&acc)[P], const float (&sc)[P], const RowConst &rc) {
  float f = 0.0f;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const float val = digits_to_float(acc[p][3] - rc.rs[3], acc[p][2] - rc.rs[2], acc[p][1] - rc.rs[1],
                                      acc[p][0] - rc.rs[0], rc.exp);
    float t = __fmul_rn(val, sc[p]);
    f = p == 0 ? t : __fadd_rn(f, t);
  }
  return f;
}

// Finish one lane's 4 accumulator registers for every plane, with preloaded constants. Rows that
// take the exact fallback are left alone here: exact_rows() writes them afterwards.
template <int P, typename PR>
__device__ __forceinline__ void flow_epilogue(const PR &pr, int n, int rowbase, const v4i (&acc)[P],
                                              const float (&sc)[P], const RowConst &rc) {
  if (pr.out_dtype == TK_I32) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = rowbase + r;
      if (m < pr.R) gstore((int32_t *)pr.out + (size_t)m * pr.n + n, acc[0][r] - rc.rs[r]);
    }
    return;
  }
  if (pr.mode == TK_MODE_INT8) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = rowbase + r;
      if (m >= pr.R || (rc.flag & (1u << r))) continue;
      store_out(pr.out, pr.out_dtype, (size_t)m * pr.n + n,
                with_residual(pr.residual, pr.out_dtype, (size_t)m * pr.n + n, int8_value<P>(acc, r, sc, rc, pr.act_scale != nullptr)));
    }
  } else {
    const int tok = rowbase >> 2;
    if (tok >= pr.M || rc.flag) return;
    store_out(pr.out, pr.out_dtype, (size_t)tok * pr.n + n,
              with_residual(pr.residual, pr.out_dtype, (size_t)tok * pr.n + n, digits_value<P>(acc, sc, rc)));
  }
}

// The epilogue of the decode kernels' second operand order (int8 contract): the lane holds token m and the four output
// channels n0 .. n0+3 in the four accumulator registers of every plane. The arithmetic per output is int8_value's, so the
// bits are those of flow_epilogue; the four results leave as one 8-byte (bf16) or 16-byte (f32) store when the row
// stride and the base address allow it and there is no residual to add. A flagged token (NaN/Inf in its activations) is
// recomputed per output in the reference's order, like exact_rows does.
template <int P, typename PR>
__device__ __forceinline__ void flow_epilogue_swapped(const PR &hot, const TkProblem &pr, int m, int n0, const v4i (&acc)[P],
                                                      const float (&sc4)[P][4], int rs, float as, unsigned flagged) {
  if (m >= hot.R) return;
  const size_t idx = (size_t)m * (size_t)hot.n + (size_t)n0;
  if (hot.out_dtype == TK_I32) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (n0 + r < hot.n) gstore((int32_t *)hot.out + idx + r, acc[0][r] - rs);
    return;
  }
  if (flagged) {
    for (int r = 0; r < 4; ++r) {
      if (n0 + r >= hot.n) break;
      float f = 0.0f;
      for (int p = 0; p < pr.planes; ++p) {
        const float t = __fmul_rn(seq_dot(pr, p, n0 + r, m, 1), pr.scales[p][n0 + r]);
        f = p == 0 ? t : __fadd_rn(f, t);
      }
      if (pr.act_scale) f = __fmul_rn(f, pr.act_scale[m]);
      store_out(hot.out, hot.out_dtype, idx + r, with_residual(hot.residual, hot.out_dtype, idx + r, f));
    }
    return;
  }
  const bool has_as = hot.act_scale != nullptr;
  float f[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    f[r] = 0.0f;
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const float t = __fmul_rn((float)(acc[p][r] - rs), sc4[p][r]);
      f[r] = p == 0 ? t : __fadd_rn(f[r], t);
    }
    if (has_as) f[r] = __fmul_rn(f[r], as);
  }
  const bool bf16 = hot.out_dtype == TK_BF16;
  const unsigned esz = bf16 ? 2u : 4u;
  const bool wide = !hot.residual && n0 + 3 < hot.n && (((uintptr_t)hot.out + idx * esz) & (bf16 ? 7u : 15u)) == 0;
  if (wide) {
    if (bf16) {
      const uint32_t lo = (uint32_t)f32_to_bf16_rne(f[0]) | ((uint32_t)f32_to_bf16_rne(f[1]) << 16);
      const uint32_t hi = (uint32_t)f32_to_bf16_rne(f[2]) | ((uint32_t)f32_to_bf16_rne(f[3]) << 16);
      typedef unsigned v2u_ __attribute__((ext_vector_type(2)));
      *(TK_GLOBAL v2u_ *)((uint16_t *)hot.out + idx) = v2u_{lo, hi};
    } else {
      typedef float v4f_ __attribute__((ext_vector_type(4)));
      *(TK_GLOBAL v4f_ *)((float *)hot.out + idx) = v4f_{f[0], f[1], f[2], f[3]};
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (n0 + r < hot.n) store_out(hot.out, hot.out_dtype, idx + r, with_residual(hot.residual, hot.out_dtype, idx + r, f[r]));
}

// The rows of one lane that hold NaN/Inf: recomputed in the reference's order (needs no accumulator).
__device__ __forceinline__ void exact_rows(const TkProblem &pr, int n, int rowbase, unsigned flag) {
  if (pr.out_dtype == TK_I32) return;
  if (pr.mode == TK_MODE_INT8) {
    for (int r = 0; r < 4; ++r) {
      const int m = rowbase + r;
      if (m >= pr.R || !(flag & (1u << r))) continue;
      float f = 0.0f;
      for (int p = 0; p < pr.planes; ++p) {
        float t = __fmul_rn(seq_dot(pr, p, n, m, 1), pr.scales[p][n]);
        f = p == 0 ? t : __fadd_rn(f, t);
      }
      if (pr.act_scale) f = __fmul_rn(f, pr.act_scale[m]);
      store_out(pr.out, pr.out_dtype, (size_t)m * pr.n + n, with_residual(pr.residual, pr.out_dtype, (size_t)m * pr.n + n, f));
    }
  } else {
    const int tok = rowbase >> 2;
    if (tok >= pr.M || !flag) return;
    float f = 0.0f;
    for (int p = 0; p < pr.planes; ++p) {
      float t = __fmul_rn(seq_dot(pr, p, n, tok, 0), pr.scales[p][n]);
      f = p == 0 ? t : __fadd_rn(f, t);
    }
    store_out(pr.out, pr.out_dtype, (size_t)tok * pr.n + n, with_residual(pr.residual, pr.out_dtype, (size_t)tok * pr.n + n, f));
  }
}

// ------------------------------------------------------------------------------------------
// operand-row pieces (shared by the activation prep kernels and the kernels that quantize themselves)
// ------------------------------------------------------------------------------------------

// A thread of the prep kernels builds whole 16-byte pieces of the operand layout. Piece q of K block
// kb (q = c*8 + h*4 + j, lane group g = 2c + h) holds the elements kb*256 + c*128 + s*32 + h*16 + j*4
// + b for s, b = 0..3: consecutive q walk 32 consecutive elements for each s, so the four loads of
// a wave are contiguous runs.
__device__ __forceinline__ size_t piece_elem0(size_t kb, int q) {
  const int c = q >> 3, h = (q >> 2) & 1, j = q & 3;
  return kb * 256 + (size_t)c * 128 + (size_t)h * 16 + (size_t)j * 4;
}
__device__ __forceinline__ size_t piece_offset(size_t kb, int q, size_t R, size_t row) {
  const int c = q >> 3, h = (q >> 2) & 1, j = q & 3, g = c * 2 + h;
  return (((kb * 4 + j) * 4 + g) * R + row) * 16;
}

__device__ __forceinline__ int wave_sum(int v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// Rows of whole K blocks, 16-byte aligned, of one element type (FAST 1 = f32, 2 = bf16): the 16 elements of the piece
// that starts at element e0 of the row at `base`, without bound, alignment or type tests.
template <int FAST>
__device__ __forceinline__ void load_piece_fast(const void *act, size_t base, size_t e0, float (&v)[16]) {
#pragma unroll
  for (int sl = 0; sl < 4; ++sl) {
    if constexpr (FAST == 2) {
      typedef unsigned v2u __attribute__((ext_vector_type(2)));
      const v2u u = *(const TK_GLOBAL v2u *)((const uint16_t *)act + base + e0 + sl * 32);
      v[sl * 4 + 0] = __uint_as_float(u.x << 16);
      v[sl * 4 + 1] = __uint_as_float(u.x & 0xFFFF0000u);
      v[sl * 4 + 2] = __uint_as_float(u.y << 16);
      v[sl * 4 + 3] = __uint_as_float(u.y & 0xFFFF0000u);
    } else {
      const v4u u = *(const TK_GLOBAL v4u *)((const float *)act + base + e0 + sl * 32);
      v[sl * 4 + 0] = __uint_as_float(u.x);
      v[sl * 4 + 1] = __uint_as_float(u.y);
      v[sl * 4 + 2] = __uint_as_float(u.z);
      v[sl * 4 + 3] = __uint_as_float(u.w);
    }
  }
}

