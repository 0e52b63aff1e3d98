// gfx950 (CDNA4) kernels for the packed ternary linear layer.
//
// Everything that contracts goes through v_mfma_i32_16x16x64_i8:
//   * weights stay 2-bit packed in HBM and in registers; one dword (16 trits of one output row)
//     becomes one 16-byte MFMA B operand with four shift+and pairs, as codes {0,1,2} = trit+1.
//     The "+1" is undone with the identity  Σ_k (code-1)·a = Σ_k code·a − Σ_k a  (per-row sum Σa
//     is produced once by the activation prep kernels).
//   * int8 activations (the W1.58A8 decode/prefill path) are MFMA A operands directly: the int32
//     accumulators are exact.
//   * float activations (f32 / bf16) are split per token into four balanced base-256 digits of a
//     31-bit fixed-point number against the token's own power-of-two exponent; the four digit rows
//     ride in the four accumulator registers of one lane, and are recombined exactly in f64.
//     The result is the exactly-rounded sum of the fixed-point values: tighter than the f32
//     k-order fold it is compared with. Tokens holding NaN/Inf take an in-kernel sequential
//     fallback that walks k in order with one f32 accumulator, like the reference does.
//
// Compiled with -ffp-contract=off: the epilogue multiplies must round exactly as the CPU's do.

#include <cstdlib>

#include "tk_internal.h"

#include "tk_device.h"


// ------------------------------------------------------------------------------------------
// decode GEMV ("skinny"): R <= 16*RT operand rows, one workgroup per 16-row output tile.
// The four waves split the K blocks; each streams 1 KiB weight chunks with one 128-bit load per
// lane, expands, and issues MFMAs against A operands held in LDS.
// ------------------------------------------------------------------------------------------

// FUSED (one row tile, a single problem whose operand rows fit LDS in one pass): the kernel builds the operand rows
// of its one to four tokens itself from pr.raw_act -- see fused_stage_rows -- and the call is one launch instead of
// two; the row constants sit in LDS behind the rows.
__device__ __forceinline__ void fused_stage_rows(const TkProblem &pr, uint4 *rows, uint8_t *cst);
__device__ __forceinline__ RowConst row_const_from_lds(const uint8_t *cst, int mode, int R, int M, int rowbase);
__device__ __forceinline__ void exact_rows_fused(const TkProblem &pr, int n, int rowbase, unsigned flag, const uint8_t *cst);
template <int P, int RT, bool FUSED = false>
__global__ __launch_bounds__(TK_WG) void tk_skinny_kernel(TkProblem single, const TkProblem *__restrict__ table,
                                                          int nprobs) {
  static_assert(!FUSED || RT == 1, "the fused form: one row tile");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tile = blockIdx.x;
  const TkProblem *prp = &single;
  if (table) {
    int lo = 0, hi = nprobs - 1;  // last problem with tile_begin <= tile
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (table[mid].tile_begin <= tile) lo = mid; else hi = mid - 1;
    }
    prp = &table[lo];
  }
  const TkProblem &pr = *prp;
  const int t = tile - pr.tile_begin;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int nb = pr.nb, R = pr.R, kc = pr.kc;

  v4i acc[P][RT];
#pragma unroll
  for (int p = 0; p < P; ++p)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[p][rt] = v4i{0, 0, 0, 0};

  const uint4 *ap4 = (const uint4 *)pr.ap;
  uint4 *lds4 = (uint4 *)smem;

  if constexpr (FUSED) {
    // The rows fit LDS in one pass (kc >= nb). A workgroup stages them once and then takes pr.run_tiles consecutive
    // output tiles (its index counts workgroups, not tiles: tile_begin is in those units), so that launches of more
    // than two tiles per CU do not repeat the tokens' prep in every tile; the reduction's buffer lies behind the rows,
    // the row constants and the norm's scratch, which all stay in place for the next tile.
    const size_t rows_bytes = (size_t)nb * 256 * R;
    uint8_t *const cst = smem + rows_bytes;
    v4i *const red = (v4i *)(cst + 1024 + (pr.norm_kind ? (size_t)pr.k * 4 + 1024 : 0));
    fused_stage_rows(pr, lds4, cst);
    const int tpw = pr.run_tiles > 0 ? pr.run_tiles : 1;
    for (int tt = 0; tt < tpw; ++tt) {
      const int tf = t * tpw + tt;
      if (tf >= pr.n_tiles) break;  // (uniform over the workgroup)
#pragma unroll
      for (int p = 0; p < P; ++p) acc[p][0] = v4i{0, 0, 0, 0};
      uint4 w[P], wn[P];
      if (wave < nb) {
#pragma unroll
        for (int p = 0; p < P; ++p) wn[p] = *(const uint4 *)(pr.codes[p] + (((size_t)tf * nb + wave) * 64 + lane) * 16);
      }
      for (int kbl = wave; kbl < nb; kbl += 4) {
        const int kn = kbl + 4 < nb ? kbl + 4 : kbl;
#pragma unroll
        for (int p = 0; p < P; ++p) {
          w[p] = wn[p];
          wn[p] = *(const uint4 *)(pr.codes[p] + (((size_t)tf * nb + kn) * 64 + lane) * 16);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint4 q = make_uint4(0, 0, 0, 0);
          if (i < R) q = lds4[((kbl * 4 + j) * 4 + g) * R + i];
          const v4i a = v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w};
#pragma unroll
          for (int p = 0; p < P; ++p) {
            const uint32_t wj = j == 0 ? w[p].x : (j == 1 ? w[p].y : (j == 2 ? w[p].z : w[p].w));
            acc[p][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, expand_codes(wj), acc[p][0], 0, 0, 0);
          }
        }
      }
      __syncthreads();  // (the first wave has finished the previous tile's epilogue, which reads `red`)
#pragma unroll
      for (int p = 0; p < P; ++p) red[(wave * P + p) * 64 + lane] = acc[p][0];
      __syncthreads();
      const int n = tf * 16 + i;
      if (wave == 0 && n < pr.n) {
        const int rowbase = 4 * g;
        v4i sum[P];
        float sc[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
          sum[p] = red[(0 * P + p) * 64 + lane];
#pragma unroll
          for (int w2 = 1; w2 < 4; ++w2) sum[p] += red[(w2 * P + p) * 64 + lane];
          sc[p] = pr.scales[p][n];
        }
        const RowConst rc = row_const_from_lds(cst, pr.mode, R, pr.M, rowbase);
        flow_epilogue<P>(pr, n, rowbase, sum, sc, rc);
        if (rc.flag) exact_rows_fused(pr, n, rowbase, rc.flag, cst);
      }
    }
    return;
  }
  for (int kb0 = 0; kb0 < nb; kb0 += kc) {
    const int kcn = min(kc, nb - kb0);
    __syncthreads();
    const int cnt = kcn * 16 * R;  // 16-byte pieces in this K chunk
    const uint4 *src = ap4 + (size_t)kb0 * 16 * R;
    for (int idx = threadIdx.x; idx < cnt; idx += TK_WG) lds4[idx] = src[idx];
    __syncthreads();

    // the chunk of the next trip is requested before this trip's arithmetic (the last trip asks for its own chunk
    // again: a cache hit), so that a wave's round trips to memory overlap with its matrix work
    uint4 w[P], wn[P];
    if (wave < kcn) {
#pragma unroll
      for (int p = 0; p < P; ++p)
        wn[p] = gload16(pr.codes[p] + (((size_t)t * nb + kb0 + wave) * 64 + lane) * 16);
    }
    for (int kbl = wave; kbl < kcn; kbl += 4) {
      const int kn = kbl + 4 < kcn ? kbl + 4 : kbl;
#pragma unroll
      for (int p = 0; p < P; ++p) {
        w[p] = wn[p];
        wn[p] = gload16(pr.codes[p] + (((size_t)t * nb + kb0 + kn) * 64 + lane) * 16);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i a[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const int row = rt * 16 + i;
          uint4 q = make_uint4(0, 0, 0, 0);
          if (row < R) q = lds4[((kbl * 4 + j) * 4 + g) * R + row];
          a[rt] = v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w};
        }
#pragma unroll
        for (int p = 0; p < P; ++p) {
          const uint32_t wj = j == 0 ? w[p].x : (j == 1 ? w[p].y : (j == 2 ? w[p].z : w[p].w));
          const v4i b = expand_codes(wj);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            acc[p][rt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[rt], b, acc[p][rt], 0, 0, 0);
        }
      }
    }
  }

  // cross-wave reduction through LDS
  __syncthreads();
  v4i *red = (v4i *)smem;
#pragma unroll
  for (int p = 0; p < P; ++p)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) red[((wave * P + p) * RT + rt) * 64 + lane] = acc[p][rt];
  __syncthreads();

  const int n = t * 16 + i;
  for (int rt = wave; rt < RT; rt += 4) {
    const int rowbase = rt * 16 + 4 * g;
    float out[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < P; ++p) {
      v4i v = red[((0 * P + p) * RT + rt) * 64 + lane];
#pragma unroll
      for (int w2 = 1; w2 < 4; ++w2) v += red[((w2 * P + p) * RT + rt) * 64 + lane];
      if (n < pr.n) {
        if (pr.out_dtype == TK_I32) {
          if (p == 0) store_raw(pr, n, rowbase, v);
        } else {
          fold_plane(pr, p, n, rowbase, v, out, p == 0);
        }
      }
    }
    if (n < pr.n && pr.out_dtype != TK_I32) finish_lane(pr, n, rowbase, out);
  }
}

// ------------------------------------------------------------------------------------------
// decode GEMV, streaming form: used when a launch holds enough output tiles to fill the chip
// (grouped launches, wide layers). A workgroup owns 4*TW consecutive 16-row tiles; each wave owns
// TW of them outright, so there is no cross-wave reduction, and every wave walks contiguous
// 1 KiB chunks of its tiles with the next K block's chunks already in flight. The activation
// operand rows stay resident in LDS for all tiles of the workgroup.
// ------------------------------------------------------------------------------------------

template <int P, int RT, int TW>
__global__ __launch_bounds__(TK_WG) void tk_stream_kernel(TkProblem single, const TkProblem *__restrict__ table,
                                                          const int *__restrict__ wg_prob) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const TkProblem *prp = &single;
  if (table) prp = &table[wg_prob[blockIdx.x]];
  const TkProblem &pr = *prp;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int nb = pr.nb, R = pr.R, kc = pr.kc;
  const int tile0 = ((blockIdx.x - pr.group_begin) * 4 + wave) * TW;

  const uint8_t *wp[TW][P];
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    // tiles past the end re-read the last tile (results discarded) so every load stays in bounds
    const int t = min(tile0 + tw, pr.n_tiles - 1);
#pragma unroll
    for (int p = 0; p < P; ++p) wp[tw][p] = pr.codes[p] + ((size_t)t * nb * 64 + lane) * 16;
  }

  v4i acc[TW][P][RT];
#pragma unroll
  for (int tw = 0; tw < TW; ++tw)
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) acc[tw][p][rt] = v4i{0, 0, 0, 0};

  const uint4 *ap4 = (const uint4 *)pr.ap;
  uint4 *lds4 = (uint4 *)smem;
  uint4 wc[TW][P], wn[TW][P];

  if (nb > 0) {
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int p = 0; p < P; ++p) wc[tw][p] = *(const uint4 *)(wp[tw][p]);
  }

  for (int kb0 = 0; kb0 < nb; kb0 += kc) {
    const int kcn = min(kc, nb - kb0);
    __syncthreads();
    const int cnt = kcn * 16 * R;
    const uint4 *src = ap4 + (size_t)kb0 * 16 * R;
    for (int idx = threadIdx.x; idx < cnt; idx += TK_WG) lds4[idx] = src[idx];
    __syncthreads();

    for (int kbl = 0; kbl < kcn; ++kbl) {
      const int kb = kb0 + kbl;
      if (kb + 1 < nb) {
#pragma unroll
        for (int tw = 0; tw < TW; ++tw)
#pragma unroll
          for (int p = 0; p < P; ++p) wn[tw][p] = *(const uint4 *)(wp[tw][p] + (size_t)(kb + 1) * TK_CHUNK_BYTES);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i a[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const int row = rt * 16 + i;
          uint4 q = make_uint4(0, 0, 0, 0);
          if (row < R) q = lds4[((kbl * 4 + j) * 4 + g) * R + row];
          a[rt] = v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w};
        }
#pragma unroll
        for (int tw = 0; tw < TW; ++tw)
#pragma unroll
          for (int p = 0; p < P; ++p) {
            const uint4 w = wc[tw][p];
            const uint32_t wj = j == 0 ? w.x : (j == 1 ? w.y : (j == 2 ? w.z : w.w));
            const v4i b = expand_codes(wj);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              acc[tw][p][rt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[rt], b, acc[tw][p][rt], 0, 0, 0);
          }
      }
#pragma unroll
      for (int tw = 0; tw < TW; ++tw)
#pragma unroll
        for (int p = 0; p < P; ++p) wc[tw][p] = wn[tw][p];
    }
  }

#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    const int t = tile0 + tw;
    const int n = t * 16 + i;
    if (t >= pr.n_tiles || n >= pr.n) continue;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int rowbase = rt * 16 + 4 * g;
      if (pr.out_dtype == TK_I32) {
        store_raw(pr, n, rowbase, acc[tw][0][rt]);
      } else {
        float out[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < P; ++p) fold_plane(pr, p, n, rowbase, acc[tw][p][rt], out, p == 0);
        finish_lane(pr, n, rowbase, out);
      }
    }
  }
}

#include "tk_flow.h"

// ------------------------------------------------------------------------------------------
// Block-scale additive planes (SALT, crates/tritium-format/src/salt.rs:1-19): every plane is a
// TQ2_0 row whose per-256-block f16 scale counts, W[n,k] = sum_p s_p[n, k/256] * trit_p[n,k], and
// out[m,n] = sum_k act[m,k] * W[n,k] on float activations. Host definition: dequantize the row (planes
// added in order, f32), then one f32 accumulator over k (crates/tritium-nn/src/layers/packed_salt.rs:
// 585-628); the reference's own GPU kernel is held to 1e-4 of that
// (crates/tritium-cuda/kernels/tq2_0_add.cu:640-719).
// ------------------------------------------------------------------------------------------

// The host's order, exactly: used for launches the flow form does not take and for tokens holding
// NaN or Inf.
__device__ __noinline__ float salt_exact_dot(const TkProblem &pr, int n, int tok) {
  const int nb = pr.nb, kdim = pr.k, planes = pr.planes;
  const size_t tile_base = (size_t)(n >> 4) * nb;
  float acc = 0.0f;
  for (int kb = 0; kb < nb; ++kb) {
    float sc[TK_MAX_PLANES];
    for (int p = 0; p < planes; ++p) sc[p] = pr.bscale[p][(tile_base + kb) * 16 + (n & 15)];
    const int kend = min(kdim, (kb + 1) * 256);
    for (int k = kb * 256; k < kend; ++k) {
      float w = 0.0f;
      for (int p = 0; p < planes; ++p) w = __fadd_rn(w, __fmul_rn(sc[p], (float)(code_at(pr.codes[p], nb, n, k) - 1)));
      acc = __fadd_rn(acc, __fmul_rn(load_act(pr.raw_act, pr.raw_dtype, (size_t)tok * kdim + k), w));
    }
  }
  return acc;
}

__global__ __launch_bounds__(TK_WG) void tk_salt_seq_kernel(TkProblem pr) {
  size_t idx = (size_t)blockIdx.x * TK_WG + threadIdx.x;
  size_t total = (size_t)pr.M * pr.n;
  if (idx >= total) return;
  store_out(pr.out, pr.out_dtype, idx, salt_exact_dot(pr, (int)(idx % pr.n), (int)(idx / pr.n)));
}

// Flow form: the stream, ring and LDS-resident operand rows of tk_flow_kernel (one run per wave),
// float activations as four digit rows per token. What differs is that a K block
// is finished on its own: after its four MFMA steps the lane turns the block's integer sums into
// the token's value (minus the block's operand-row sums, which stand in for code = trit + 1),
// multiplies by the block scale of its output column and adds that to a float accumulator; the
// integer accumulators start again from zero. Per block: exact up to 1.5 ulp; the f32 sum over
// blocks and planes is what the 1e-4 bound covers.
template <int P, int RT, int DR>
__global__ __launch_bounds__(512) void tk_salt_flow_kernel(const TkProblem single) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const TkProblem &pr = *single_problem();
  constexpr int D = DR - 1;
  const int NW = (int)(blockDim.x >> 6);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int nb = pr.nb, R = pr.R, S = pr.run_tiles, n_tiles = pr.n_tiles, M = pr.M, ncols = pr.n;
  const int out_dtype = pr.out_dtype;
  void *const out = pr.out;
  const uint8_t *codes[P];
  const float *bscale[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    codes[p] = pr.codes[p];
    bscale[p] = pr.bscale[p];
  }
  const int nbpad = (nb + DR - 1) / DR * DR;
  const int first = (blockIdx.x * NW + wave) * S;
  const unsigned plane_last = (unsigned)n_tiles * (unsigned)nb - 1u;
  unsigned roff = (unsigned)first * (unsigned)nb * 1024u + (unsigned)lane * 16u;
  const unsigned run_last = (unsigned)(first + S - 1) * (unsigned)nb + (unsigned)nb - 1u;
  const unsigned last_off = min(run_last, plane_last) * 1024u + (unsigned)lane * 16u;

  uint4 ring[DR][P];
  float ring_s[DR][P];
  auto request = [&](int slot, bool real) {
    const unsigned off = min(roff, last_off);
#pragma unroll
    for (int p = 0; p < P; ++p) {
      ring[slot][p] = gload16_stream(codes[p] + (size_t)off);
      ring_s[slot][p] = gload(bscale[p] + (size_t)(off >> 10) * 16 + i);  // chunk index * 16 + column
    }
    roff += real ? 1024u : 0u;
  };
#pragma unroll
  for (int d = 0; d < D; ++d) request(d, d < nb);

  // operand rows, then the per-block row sums behind them
  int *lds_bs = (int *)(smem + (size_t)nb * 256 * R);
  {
    const uint4 *ap4 = (const uint4 *)pr.ap;
    uint4 *lds4w = (uint4 *)smem;
    const int cnt = nb * 16 * R;
    for (int idx = threadIdx.x; idx < cnt; idx += (int)blockDim.x) lds4w[idx] = gload16(ap4 + idx);
    for (int idx = threadIdx.x; idx < nb * R; idx += (int)blockDim.x) lds_bs[idx] = gload(pr.blocksum + idx);
  }
  int exps[RT];
  unsigned flag[RT];
  unsigned any_flag = 0;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int tok = rt * 4 + g;
    exps[rt] = tok < M ? gload(pr.exps + tok) : 0;
    flag[rt] = tok < M && pr.flags ? gload(pr.flags + tok) : 0u;
    any_flag |= flag[rt];
  }
  __syncthreads();
  const uint4 *lds4 = (const uint4 *)smem;
  int arow[RT], srow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    arow[rt] = min(rt * 16 + i, R - 1);
    srow[rt] = min(rt * 16 + 4 * g, R - 4);  // R is a multiple of 4 (four digit rows per token)
  }

  for (int s = 0; s < S; ++s) {
    v4i acc[RT][P];
    float facc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) facc[rt] = 0.0f;
    int kbg = 0;
    do {
#pragma unroll
      for (int d = 0; d < DR; ++d) {
        const int kb = kbg + d;
        {
          int kb2 = kb + D;
          if (kb2 >= nbpad) kb2 -= nbpad;
          request((d + D) % DR, kb2 < nb);
        }
        if (kb < nb) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v4i a[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
              const uint4 q = lds4[((kb * 4 + j) * 4 + g) * R + arow[rt]];
              a[rt] = v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w};
            }
#pragma unroll
            for (int p = 0; p < P; ++p) {
              const uint4 w = ring[d][p];
              const uint32_t wj = j == 0 ? w.x : (j == 1 ? w.y : (j == 2 ? w.z : w.w));
              const v4i b = expand_codes(wj);
#pragma unroll
              for (int rt = 0; rt < RT; ++rt)  // the first step of a block starts from zero
                acc[rt][p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[rt], b, j == 0 ? v4i{0, 0, 0, 0} : acc[rt][p], 0, 0, 0);
            }
          }
          // finish the block: the token's dot product over these 256 k in units of its grid (the
          // power of two is applied once, after the last block), times the block scale
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            const v4i rs = *(const v4i *)(lds_bs + kb * R + srow[rt]);
#pragma unroll
            for (int p = 0; p < P; ++p) {
              const float v = digits_to_float(acc[rt][p][3] - rs[3], acc[rt][p][2] - rs[2], acc[rt][p][1] - rs[1],
                                              acc[rt][p][0] - rs[0], 0);
              facc[rt] = __fadd_rn(facc[rt], __fmul_rn(v, ring_s[d][p]));
            }
          }
        }
      }
      kbg += DR;
    } while (kbg < nbpad);

    const int t = first + s, n = t * 16 + i;
    if (t < n_tiles && n < ncols) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int tok = rt * 4 + g;
        if (tok < M && !flag[rt]) store_out(out, out_dtype, (size_t)tok * ncols + n, ldexpf(facc[rt], exps[rt]));
      }
      if (any_flag) {
        for (int rt = 0; rt < RT; ++rt) {
          const int tok = rt * 4 + g;
          if (tok < M && flag[rt]) store_out(out, out_dtype, (size_t)tok * ncols + n, salt_exact_dot(pr, n, tok));
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// prefill GEMM. Workgroup tile = 64 operand rows x (TK_GEMM_WAVES waves * NT tiles * 16 outputs),
// all P planes of a tile in the same wave (P*NT = 4 accumulator tiles per row tile, so one LDS read
// of an A operand feeds 4 MFMAs). A blocks of 256 k travel global -> LDS by DMA into three slots,
// two blocks ahead of the MFMAs; the 2-bit weight chunks of the wave's own tiles go straight to
// registers (never through LDS), also two blocks ahead, and a dword is expanded into an MFMA operand
// when needed; one barrier per block. A single wave cannot keep the MFMA pipe full (measured: ~25
// cycles per 16x16x64 issue from one wave, ~18 from two), and waves of one workgroup stall
// together at its barrier, so the kernel is sized for several independent workgroups per CU.
// ------------------------------------------------------------------------------------------

#ifndef TK_GEMM_WAVES
#define TK_GEMM_WAVES 4
#endif
#define TK_GEMM_THREADS (TK_GEMM_WAVES * 64)

#ifndef TK_GEMM_OCC
#define TK_GEMM_OCC 3
#endif

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt[3:0] | [15:14])
#define TK_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

template <int P, int NT>
__device__ __forceinline__ void tk_gemm_epilogue(const TkProblem &pr, const TkHot &hot, const float *const (&scales)[P],
                                                 v4i (&acc)[4][NT * P], uint8_t *smem, int tid, int bm, int bn);

// TABLE: a grouped launch; the workgroup finds its problem through wg_prob and counts its position
// from the problem's first workgroup (a multiple of 8, so the XCD of a workgroup is unchanged).
template <int P, int NT, bool TABLE>
__global__ __launch_bounds__(TK_GEMM_THREADS) __attribute__((amdgpu_waves_per_eu(TK_GEMM_OCC, TK_GEMM_OCC))) void
tk_gemm_kernel(const TkProblem single, const TkProblem *__restrict__ table, const int *__restrict__ wg_prob) {
  const TkProblem &pr = TABLE ? table[wg_prob[blockIdx.x]] : single;
  // local copies: a field read through the table pointer would be fetched again after every store
  const TkHot hot = make_hot(pr);
  const uint8_t *codes[P];
  const float *scales[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    codes[p] = pr.codes[p];
    scales[p] = pr.scales[p];
  }
  const int8_t *ap = pr.ap;
  const int rs = pr.rs, n_tiles = pr.n_tiles;
  const unsigned wg = blockIdx.x - (TABLE ? (unsigned)pr.group_begin : 0u);
  constexpr int RT = 4, ROWS = RT * 16, A4 = 16 * ROWS, NB = NT * P;
  constexpr int SEGS = 16 / TK_GEMM_WAVES;  // 1-KiB A segments (one (j,g) pair x 64 rows) per wave per block
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // three A blocks of 16 KiB
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int nb = pr.nb, R = pr.R;
  // XCD-aware tile order: consecutive workgroup ids go round-robin to the 8 XCDs, each with its own
  // L2. XCD x = id % 8 gets a compact sub-grid of sub_m x sub_n tiles, so the A row blocks and the
  // weight column blocks it touches stay resident in that L2 instead of every XCD streaming all.
  const int xcd = wg & 7, slot = wg >> 3;
  const int bm = (xcd % pr.xr) * pr.sub_m + slot % pr.sub_m;
  const int bn = (xcd / pr.xr) * pr.sub_n + slot / pr.sub_m;
  if (bm >= pr.grid_m || bn >= pr.grid_n) return;
  const int row0 = bm * ROWS;
  const int tile0 = (bn * TK_GEMM_WAVES + wave) * NT;

  // weight chunk offsets inside a plane (tiles past the end re-read the last tile; results dropped)
  unsigned woff[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) woff[nt] = ((unsigned)min(tile0 + nt, n_tiles - 1) * (unsigned)nb * 64u + lane) * 16u;

  // A rows travel global -> LDS directly (no registers): one wave-wide 16-byte-per-lane load lands
  // as 1 KiB at a wave-uniform LDS address, which is exactly one (j,g) segment of 64 rows. Rows past
  // R are clamped to the last row (their results are never stored).
  const unsigned a_lane = (unsigned)min(row0 + lane, R - 1) * 16u;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto dma_block = [&](int kb, int slot3) {
#pragma unroll
    for (int u = 0; u < SEGS; ++u) {
      const int seg = wave_u * SEGS + u;
      const uint8_t *seg_base = (const uint8_t *)ap + ((size_t)kb * 16 + seg) * (size_t)rs * 16;  // wave-uniform
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(seg_base + a_lane),
                                       (__attribute__((address_space(3))) void *)(smem + ((size_t)slot3 * A4 + (size_t)seg * ROWS) * 16),
                                       16, 0, 0);
    }
  };

  // Per-row constants of the tile (row sums, activation scales or grid exponents, fallback flags)
  // travel to LDS by DMA now, one kind per wave, into 1 KiB past the A slots: the epilogue reads
  // them from there, so they neither wait on memory then nor occupy registers during the main loop.
  // Indices past the end are clamped; what is read for them is never used.
  constexpr int CST = 3 * A4 * 16;  // int rs[64] | float as[64] | int exp[64] | uint flag[64]
  {
    const bool int8_in = hot.mode == TK_MODE_INT8;
    const int row_c = min(row0 + lane, R - 1), tok_c = min((row0 >> 2) + lane, hot.M - 1);
    const void *src = nullptr;
    if (wave_u == 0) src = hot.rowsum + row_c;
    else if (wave_u == 1) src = (int8_in && hot.act_scale) ? (const void *)(hot.act_scale + row_c) : nullptr;
    else if (wave_u == 2) src = int8_in ? nullptr : (const void *)(hot.exps + tok_c);
    else if (wave_u == 3) src = hot.flags ? (const void *)(hot.flags + (int8_in ? row_c : tok_c)) : nullptr;
    if (src && wave_u < 4)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                       (__attribute__((address_space(3))) void *)(smem + CST + wave_u * 256), 4, 0, 0);
  }

  v4i acc[RT][NB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int x = 0; x < NB; ++x) acc[rt][x] = v4i{0, 0, 0, 0};

  // The operand loads of the main loop are written as asm, with explicit waits. The compiler's own
  // wait insertion cannot keep loads in flight across this loop: it does not see that an LDS read
  // of slot `cur` never aliases the DMA into another slot, and with DMA and register loads pending
  // together it drains the whole vector-memory counter at the first use of a loaded register --
  // right after the prefetches were issued. An empty asm with a "+v" operand after each wait ties
  // every later use of a loaded register to that wait.
  // one address register for every read: slot, k step and row tile all sit in the 16-bit offset field
  auto lds_read = [&](v4i (&a)[RT], unsigned addr, int off) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[rt]) : "v"(addr), "n"(off + rt * 256));
  };
  auto lds_wait = [&](v4i (&a)[RT]) {
    asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) asm volatile("" : "+v"(a[rt]));
  };
  auto load_w = [&](v4i (&w)[NB], int kb) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int p = 0; p < P; ++p)
        asm volatile("global_load_dwordx4 %0, %1, %2"
                     : "=v"(w[nt * P + p])
                     : "v"(woff[nt] + (unsigned)kb * (unsigned)TK_CHUNK_BYTES), "s"(codes[p]));
  };
  auto tie_w = [&](v4i (&w)[NB]) {
#pragma unroll
    for (int x = 0; x < NB; ++x) asm volatile("" : "+v"(w[x]));
  };

  // Prefetch distance is two blocks for both operands: at the top of block kb the weight chunks and
  // the A DMA of block kb+2 are issued; by the end of block kb everything of block kb+1 has landed.
  v4i wc[NB], wn[NB], wf[NB];
#pragma unroll
  for (int x = 0; x < NB; ++x) wc[x] = wn[x] = wf[x] = v4i{0, 0, 0, 0};
  if (nb > 0) {
    load_w(wc, 0);
    dma_block(0, 0);
    if (nb > 1) {
      load_w(wn, 1);
      dma_block(1, 1);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SEGS + NB));  // block 0 has landed; block 1 may be in flight
    } else {
      asm volatile("s_waitcnt vmcnt(0)");
    }
    tie_w(wc);
  }
  __builtin_amdgcn_s_barrier();

  const unsigned lds_lane = (unsigned)(size_t)(__attribute__((address_space(3))) uint8_t *)smem + (unsigned)(g * ROWS + i) * 16u;
  // One block: `w` holds its weight chunks, `w1` those of block kb+1 (in flight or landed), `w2` is
  // free and receives block kb+2. The three register sets and the three LDS slots rotate by name
  // (the loop below is unrolled by three), never by copying: a register with a load in flight must
  // not be read.
  auto block = [&](v4i (&w)[NB], v4i (&w1)[NB], v4i (&w2)[NB], int kb, int cur) {
    const bool more2 = kb + 2 < nb;
    const int nxt2 = cur == 0 ? 2 : cur - 1;  // slot of block kb+2 == slot of block kb-1, free since the last barrier
    if (more2) {
      load_w(w2, kb + 2);
      dma_block(kb + 2, nxt2);
    }
    v4i a[RT];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lds_read(a, lds_lane, cur * (A4 * 16) + j * (4 * ROWS * 16));
      lds_wait(a);
#pragma unroll
      for (int x = 0; x < NB; ++x) {
        const v4i b = expand_codes((uint32_t)w[x][j]);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[rt], b, acc[rt][x], 0, 0, 0);
      }
    }
    // Everything of block kb+1 (issued one block ago) must have landed before the barrier lets anyone
    // read it; the loads of block kb+2, the youngest of this wave, stay in flight.
    if (more2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SEGS + NB)); else asm volatile("s_waitcnt vmcnt(0)");
    tie_w(w1);
    __builtin_amdgcn_s_barrier();
  };
  int kb = 0;
  for (; kb + 3 <= nb; kb += 3) {  // one exit only: the accumulators keep their registers
    block(wc, wn, wf, kb, 0);
    block(wn, wf, wc, kb + 1, 1);
    block(wf, wc, wn, kb + 2, 2);
  }
  if (kb < nb) {
    block(wc, wn, wf, kb, 0);
    if (kb + 1 < nb) block(wn, wf, wc, kb + 1, 1);
  }

  // The epilogue derives its lane coordinates afresh from a laundered thread id: sharing them with
  // the prologue would keep a dozen registers alive across the main loop, which has none to spare.
  unsigned tid_e = threadIdx.x;
  asm volatile("" : "+v"(tid_e));
  tk_gemm_epilogue<P, NT>(pr, hot, scales, acc, smem, (int)tid_e, bm, bn);
}

template <int P, int NT>
__device__ __forceinline__ void tk_gemm_epilogue(const TkProblem &pr, const TkHot &hot, const float *const (&scales)[P],
                                                 v4i (&acc)[4][NT * P], uint8_t *smem, int tid, int bm, int bn) {
  constexpr int RT = 4, ROWS = RT * 16, A4 = 16 * ROWS, CST = 3 * A4 * 16;
  const int wave = tid >> 6, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int R = hot.R, row0 = bm * ROWS, tile0 = (bn * TK_GEMM_WAVES + wave) * NT;
  const int n_tiles = (hot.n + 15) >> 4;
  // Epilogue. The row constants are in LDS since the prologue: one 16-byte read per row tile.
  const int *cst_rs = (const int *)(smem + CST);
  const float *cst_as = (const float *)(smem + CST + 256);
  const int *cst_exp = (const int *)(smem + CST + 512);
  const int *cst_flag = (const int *)(smem + CST + 768);
  unsigned my_flag = 0;
  if (hot.flags && tid < ROWS) {
    const bool in_range = hot.mode == TK_MODE_INT8 ? row0 + tid < R : (row0 >> 2) + tid < hot.M;
    if (in_range) my_flag = cst_flag[tid] ? 1u : 0u;
  }
  float sc[NT][P];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = (tile0 + nt) * 16 + i;
#pragma unroll
    for (int p = 0; p < P; ++p) sc[nt][p] = (tile0 + nt < n_tiles && n < hot.n) ? gload(scales[p] + n) : 0.0f;
  }
  const int wg_flag = __syncthreads_or((int)my_flag);
  auto row_const = [&](int rt) {
    RowConst rc;
    const v4i rs4 = *(const v4i *)(cst_rs + rt * 16 + 4 * g);
    const float4 as4 = *(const float4 *)(cst_as + rt * 16 + 4 * g);
    rc.rs[0] = rs4.x; rc.rs[1] = rs4.y; rc.rs[2] = rs4.z; rc.rs[3] = rs4.w;
    rc.as[0] = as4.x; rc.as[1] = as4.y; rc.as[2] = as4.z; rc.as[3] = as4.w;
    rc.exp = cst_exp[rt * 4 + g];
    rc.flag = 0;
    if (wg_flag) {
      if (hot.mode == TK_MODE_INT8) {
        const v4i f4 = *(const v4i *)(cst_flag + rt * 16 + 4 * g);
        rc.flag = (f4.x ? 1u : 0u) | (f4.y ? 2u : 0u) | (f4.z ? 4u : 0u) | (f4.w ? 8u : 0u);
      } else {
        rc.flag = cst_flag[rt * 4 + g] ? 1u : 0u;
      }
    }
    return rc;
  };

  // The MFMA result layout gives a lane 16 outputs of one column, four rows apart, so a direct
  // store instruction writes 32-byte pieces of four different output rows. When the rows of the
  // output are 16-byte aligned, the finished values are staged through LDS instead (free after the
  // last barrier of the main loop) and leave as whole 16-byte pieces of contiguous row segments:
  // every store instruction of a wave then covers full cache lines.
  const int esz = hot.out_dtype == TK_BF16 ? 2 : 4;
  // (a call with a fused residual add takes the direct stores: the residual is read where the value is formed)
  const bool staged = (((size_t)hot.n * esz) & 15) == 0 && (((size_t)hot.out) & 15) == 0 && !hot.residual;
  if (staged) {
    constexpr int WG_COLS = TK_GEMM_WAVES * NT * 16;
    const bool int8_mode = hot.mode == TK_MODE_INT8 || hot.out_dtype == TK_I32;
    const int halves = esz == 4 ? 2 : 1;            // 4-byte outputs take the 64 rows in two halves
    const int rt_per_half = RT / halves;
    const int orows_rt = int8_mode ? 16 : 4;        // output rows per row tile (4 digit rows = 1 token)
    const int stride = WG_COLS * esz + 16;          // padded: the 4 lane groups of a wave hit different banks
    const int pieces_row = WG_COLS * esz / 16;      // 16-byte pieces per staged row (a power of two)
    const int out_row0 = int8_mode ? row0 : (row0 >> 2);
    const int out_rows = int8_mode ? hot.R : hot.M;
    const int col0 = bn * WG_COLS;
    const bool has_as = hot.act_scale != nullptr;
    for (int h = 0; h < halves; ++h) {
      if (h > 0) __syncthreads();
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if (rt / rt_per_half != h) continue;
        const int rl = rt - h * rt_per_half;
        const RowConst rc = row_const(rt);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const int cl = (wave * NT + nt) * 16 + i;
          v4i av[P];
#pragma unroll
          for (int p = 0; p < P; ++p) av[p] = acc[rt][nt * P + p];
          if (hot.out_dtype == TK_I32) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              *(int32_t *)(smem + (size_t)(rl * 16 + 4 * g + r) * stride + cl * 4) = av[0][r] - rc.rs[r];
          } else if (hot.mode == TK_MODE_INT8) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float f = int8_value<P>(av, r, sc[nt], rc, has_as);
              uint8_t *dst = smem + (size_t)(rl * 16 + 4 * g + r) * stride + cl * esz;
              if (esz == 2) *(uint16_t *)dst = f32_to_bf16_rne(f); else *(float *)dst = f;
            }
          } else {
            const float f = digits_value<P>(av, sc[nt], rc);
            uint8_t *dst = smem + (size_t)(rl * 4 + g) * stride + cl * esz;
            if (esz == 2) *(uint16_t *)dst = f32_to_bf16_rne(f); else *(float *)dst = f;
          }
        }
      }
      __syncthreads();
      const int rows_h = rt_per_half * orows_rt;
      const int per16 = 16 / esz;
      for (int pc = tid; pc < rows_h * pieces_row; pc += TK_GEMM_THREADS) {
        const int rl = pc / pieces_row, piece = pc - rl * pieces_row;
        const int orow = out_row0 + h * rows_h + rl;
        const int c = col0 + piece * per16;
        if (orow >= out_rows || c >= hot.n) continue;
        if (wg_flag && hot.out_dtype != TK_I32 && gload(hot.flags + orow)) continue;  // written by exact_rows below
        const uint8_t *src = smem + (size_t)rl * stride + piece * 16;
        uint8_t *dst = (uint8_t *)hot.out + ((size_t)orow * hot.n + c) * esz;
        *(TK_GLOBAL v4u *)dst = *(const v4u *)src;  // n is a multiple of per16 here, so a piece never straddles the row end
      }
    }
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const RowConst rc = row_const(rt);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int t = tile0 + nt;
        const int n = t * 16 + i;
        if (t >= n_tiles || n >= hot.n) continue;
        v4i av[P];
#pragma unroll
        for (int p = 0; p < P; ++p) av[p] = acc[rt][nt * P + p];
        flow_epilogue<P>(hot, n, row0 + rt * 16 + 4 * g, av, sc[nt], rc);
      }
    }
  }
  if (wg_flag) {
    for (int nt = 0; nt < NT; ++nt) {
      const int t = tile0 + nt;
      const int n = t * 16 + i;
      if (t >= pr.n_tiles || n >= pr.n) continue;
      for (int rt = 0; rt < RT; ++rt) {
        const int rowbase = row0 + rt * 16 + 4 * g;
        const unsigned fl = row_flags(pr, rowbase);
        if (fl) exact_rows(pr, n, rowbase, fl);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// prefill GEMM on v_mfma_i32_32x32x32_i8. Same workgroup tile, pipeline and LDS layout as the
// kernel above; the matrix instruction is the 32x32 one, which this chip sustains at 4.0 POPS where
// the 16x16x64 form stops at 3.0 (one wave per SIMD is enough to reach it). Operand mapping, with
// lane L = 32*kappa + 16*h + r:
//   B (32 weight rows x 32 k): two 16-row tiles side by side. Lane L takes its 16 bytes from tile
//     h of the pair, row r, 16-byte piece g = 2*l + kappa of that row's 64 code bytes (l = 0,1: two
//     loads per pair and K block; the device weight layout is unchanged, only the lane -> address
//     map differs). Dword j of load l expands to the operand of k step (l, j): 8 steps per block.
//   A (32 operand rows x 32 k): lane L reads piece (kb, j, g = 2*l + kappa) of row 32*rt2 + (L & 31),
//     the same 16-byte pieces the 16x16x64 kernel reads, so the operand row layout is unchanged too.
//   D: register i of lane L is row 32*rt2 + 8*(i/4) + 4*kappa + i%4, column (pair, h, r): four
//     consecutive registers are four consecutive rows, as the epilogues expect.
// The tiles of a pair belong to the same plane (tile index x = p*NT + nt, pairs (2y, 2y+1)), so the
// planes of one output meet in one lane; NT is even.
// ------------------------------------------------------------------------------------------


template <int P, int NT, int WR>
__device__ __forceinline__ void tk_gemm32_epilogue(const TkProblem &pr, const TkHot &hot, const float *const (&scales)[P],
                                                   v16i (&acc)[2 / WR][NT * P / 2], uint8_t *smem, int tid, int bm, int bn);

#ifndef TK_GEMM32_STAGES
#define TK_GEMM32_STAGES 3
#endif
#ifndef TK_GEMM_BAND
#define TK_GEMM_BAND 8
#endif
#ifndef TK_GEMM32_OCC3
#define TK_GEMM32_OCC(P) ((P) >= 3 ? 2 : 3)
#endif

// WR = 1: the four waves of a workgroup sit side by side, each over all 64 rows and its own NT tiles.
// WR = 2: two by two -- a wave takes 32 of the rows and NT tiles of one half of the columns. Per k step a
// wave then reads one 32-row A piece from LDS instead of two for the same number of matrix instructions
// (with one plane and two tiles per wave side by side -- one pair: two reads, two instructions per step --
// the four waves of a workgroup ask LDS for 128 bytes per clock at full matrix rate), and every weight
// chunk is loaded by two waves instead of one. Measured on the 64 x 128 form of the one-plane kernel,
// int8 rows in, bf16 out: 2048 x 2560 -> 6912 53.0 us side by side, 54.9 two by two; 512 tokens 20.2 /
// 21.1; 2048 x 6912 -> 2560 53.3 / 56.6. The LDS reads are not what holds that form back; the doubled
// weight loads cost more than the halved reads save. Side by side stays the default; two by two is
// kept behind a knob (identical bits).
template <int P, int NT, bool TABLE, bool KSPLIT = false, int WR = 1>
__global__ __launch_bounds__(TK_GEMM_THREADS) __attribute__((amdgpu_waves_per_eu(TK_GEMM32_OCC(P), TK_GEMM32_OCC(P)))) void
tk_gemm32_kernel(const TkProblem single, const TkProblem *__restrict__ table, const int *__restrict__ wg_prob) {
  static_assert(NT % 2 == 0, "tiles are processed in pairs");
  static_assert(WR == 1 || WR == 2, "one or two row groups");
  constexpr int WC = TK_GEMM_WAVES / WR, RT2W = 2 / WR;  // column groups; 32-row tiles per wave
  static_assert(!(TABLE && KSPLIT), "the K split is for single launches");
  const TkProblem &pr = TABLE ? table[wg_prob[blockIdx.x]] : single;
  const TkHot hot = make_hot(pr);
  const uint8_t *codes[P];
  const float *scales[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    codes[p] = pr.codes[p];
    scales[p] = pr.scales[p];
  }
  const int8_t *ap = pr.ap;
  const int rs = pr.rs, n_tiles = pr.n_tiles;
  const unsigned wg = blockIdx.x - (TABLE ? (unsigned)pr.group_begin : 0u);
  constexpr int ROWS = 64, A4 = 16 * ROWS, NB = NT * P, NP = NB / 2, HP = NT / 2;  // HP pairs per plane
  constexpr int SEGS = 16 / TK_GEMM_WAVES;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // three A blocks of 16 KiB + row constants
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, h = (lane >> 4) & 1, kappa = lane >> 5;
  const int nb_full = pr.nb, R = pr.R;
  // XCD x = id % 8 owns a compact sub-grid of sub_m x sub_n tiles. Inside it the slots walk bands of
  // TK_GEMM_BAND row tiles: down the band first, then along the columns, so the ~100 workgroups an
  // XCD holds at a time are a band x 12 patch (8 A row blocks + 12 weight column blocks to keep in
  // its L2) instead of a full column strip (32 + 3).
  // K split: the slices of a tile are consecutive slots of one XCD (they meet in its L2).
  const int ksn = KSPLIT ? pr.ksplit : 1;
  const int xcd = wg & 7, slot_k = wg >> 3;
  const int slot = KSPLIT ? slot_k / ksn : slot_k, ks = KSPLIT ? slot_k - slot * ksn : 0;
  // slice ks takes the K blocks [ks * nb / ksn, (ks + 1) * nb / ksn): at least two each (the host keeps
  // ksn <= nb / 2), so the pipeline's first two stages are loaded unconditionally
  const int kb_begin = KSPLIT ? ks * nb_full / ksn : 0;
  const int nb = KSPLIT ? (ks + 1) * nb_full / ksn - kb_begin : nb_full;
  const int sub_m = pr.sub_m, sub_n = pr.sub_n;
  const int band_sz = TK_GEMM_BAND * sub_n;
  const int band = slot / band_sz, in_band = slot - band * band_sz;
  const int band_rows = min(TK_GEMM_BAND, sub_m - band * TK_GEMM_BAND);  // the last band may be shorter
  const int lm = band * TK_GEMM_BAND + in_band % band_rows, ln = in_band / band_rows;
  const int bm = (xcd % pr.xr) * sub_m + lm;
  const int bn = (xcd / pr.xr) * sub_n + ln;
  if (lm >= sub_m || ln >= sub_n || bm >= pr.grid_m || bn >= pr.grid_n) return;
  const int row0 = bm * ROWS;
  const int wr = wave / WC, wc = wave % WC;
  const int tile0 = (bn * WC + wc) * NT;

  // per pair: this lane's address of load l = 0 in K block 0 (load 1 is 512 bytes further, block kb
  // kb KiB further); tiles past the end re-read the last tile (results dropped)
  const uint8_t *wptr[NP];
#pragma unroll
  for (int y = 0; y < NP; ++y) {
    const int p = y / HP, nt = (y % HP) * 2 + h;
    wptr[y] = codes[p] + ((size_t)min(tile0 + nt, n_tiles - 1) * (size_t)nb_full * 64 + (size_t)(kappa * 16 + r16)) * 16 +
              (size_t)kb_begin * TK_CHUNK_BYTES;
  }

  const unsigned a_lane = (unsigned)min(row0 + lane, R - 1) * 16u;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto dma_block = [&](int kb, int slot3) {
#pragma unroll
    for (int u = 0; u < SEGS; ++u) {
      const int seg = wave_u * SEGS + u;
      const uint8_t *seg_base = (const uint8_t *)ap + ((size_t)(kb_begin + kb) * 16 + seg) * (size_t)rs * 16;  // wave-uniform
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(seg_base + a_lane),
                                       (__attribute__((address_space(3))) void *)(smem + ((size_t)slot3 * A4 + (size_t)seg * ROWS) * 16),
                                       16, 0, 0);
    }
  };

  constexpr int CST = TK_GEMM32_STAGES * A4 * 16;  // int rs[64] | float as[64] | int exp[64] | uint flag[64]
  {
    const bool int8_in = hot.mode == TK_MODE_INT8;
    const int row_c = min(row0 + lane, R - 1), tok_c = min((row0 >> 2) + lane, hot.M - 1);
    const void *src = nullptr;
    if (wave_u == 0) src = hot.rowsum + row_c;
    else if (wave_u == 1) src = (int8_in && hot.act_scale) ? (const void *)(hot.act_scale + row_c) : nullptr;
    else if (wave_u == 2) src = int8_in ? nullptr : (const void *)(hot.exps + tok_c);
    else if (wave_u == 3) src = hot.flags ? (const void *)(hot.flags + (int8_in ? row_c : tok_c)) : nullptr;
    if (src && wave_u < 4)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                       (__attribute__((address_space(3))) void *)(smem + CST + wave_u * 256), 4, 0, 0);
  }

  v16i acc[RT2W][NP];
#pragma unroll
  for (int rt2 = 0; rt2 < RT2W; ++rt2)
#pragma unroll
    for (int y = 0; y < NP; ++y)
#pragma unroll
      for (int c = 0; c < 16; ++c) acc[rt2][y][c] = 0;

  // operand loads as asm with explicit waits, as in the kernel above. The compiler does not know
  // that the destination registers of such a load are in flight until the wait: were it to split
  // their live range (a copy out and back under register pressure) it would read stale data. The
  // build checks the generated code for exactly that (tritium_amd/check_isa.py) and fails on it.
  auto lds_read = [&](v4i (&a)[RT2W], unsigned addr, int off) {
#pragma unroll
    for (int rt2 = 0; rt2 < RT2W; ++rt2)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[rt2]) : "v"(addr), "n"(off + rt2 * 512));
  };
  // wait until only the RT2W reads of the next k step (`ahead`) or none are still in flight: LDS reads
  // return in order
  auto lds_wait = [&](v4i (&a)[RT2W], bool ahead) {
    if (ahead) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(RT2W));
    else asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
    for (int rt2 = 0; rt2 < RT2W; ++rt2) asm volatile("" : "+v"(a[rt2]));
  };
  // Grouped launches (decode batches: one row block per member) and K-split launches (few workgroups) read every weight
  // byte once: their loads carry the non-temporal bit, like the decode kernels' weight stream. A prefill launch reads a
  // chunk again in every row block and leaves it to the caches. (Chosen per instantiation: a branch around two forms
  // of the load would put both into the instruction stream the build's in-flight check walks.)
  constexpr bool W_ONCE = TABLE || KSPLIT;
  auto load_w = [&](v4i (&w)[NP][2], int kb) {
#pragma unroll
    for (int y = 0; y < NP; ++y) {
      const uint8_t *ptr = wptr[y] + (size_t)kb * TK_CHUNK_BYTES;
      if constexpr (W_ONCE) {
        asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(w[y][0]) : "v"(ptr));
        asm volatile("global_load_dwordx4 %0, %1, off offset:512 nt" : "=v"(w[y][1]) : "v"(ptr));
      } else {
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(w[y][0]) : "v"(ptr));
        asm volatile("global_load_dwordx4 %0, %1, off offset:512" : "=v"(w[y][1]) : "v"(ptr));
      }
    }
  };
  auto tie_w = [&](v4i (&w)[NP][2]) {
#pragma unroll
    for (int y = 0; y < NP; ++y) {
      asm volatile("" : "+v"(w[y][0]));
      asm volatile("" : "+v"(w[y][1]));
    }
  };

  // NS register sets and NS LDS slots rotate by name (the loop is unrolled NS times): block kb uses
  // set and slot kb % NS; at its top the weight chunks and the A DMA of block kb+NS-1 are issued into
  // the set and slot block kb-1 just left; at its end everything of block kb+1 must have landed,
  // the younger blocks stay in flight.
  constexpr int NS = TK_GEMM32_STAGES;
  v4i wset[NS][NP][2];
#pragma unroll
  for (int q = 0; q < NS; ++q)
#pragma unroll
    for (int y = 0; y < NP; ++y)
#pragma unroll
      for (int l = 0; l < 2; ++l) wset[q][y][l] = v4i{0, 0, 0, 0};
  // wait until at most `blocks` of the youngest issued blocks are still in flight
  auto wait_blocks = [&](int blocks) {
    if (blocks <= 0) asm volatile("s_waitcnt vmcnt(0)");
    else if (blocks == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SEGS + NB));
    else if (blocks == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (SEGS + NB)));
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * (SEGS + NB)));
  };
#pragma unroll
  for (int q = 0; q < NS - 1; ++q)
    if (KSPLIT || q < nb) {
      load_w(wset[q], q);
      dma_block(q, q);
    }
  wait_blocks(KSPLIT ? NS - 2 : min(NS - 2, nb - 1));  // block 0 has landed
#pragma unroll
  for (int q = 0; q < NS; ++q) tie_w(wset[q]);
  __builtin_amdgcn_s_barrier();

  const unsigned lds_lane = (unsigned)(size_t)(__attribute__((address_space(3))) uint8_t *)smem +
                            (unsigned)(kappa * ROWS + wr * RT2W * 32 + (lane & 31)) * 16u;
  v4i a[2][RT2W];
  auto block = [&](auto cur_c, int kb) {
    constexpr int cur = decltype(cur_c)::value, nxt = (cur + NS - 1) % NS, n1 = (cur + 1) % NS;
    if (kb + NS - 1 < nb) {
      load_w(wset[nxt], kb + NS - 1);
      dma_block(kb + NS - 1, nxt);
    }
    // the A pieces of k step s + 1 are read while the matrix instructions of step s run; those of step 0
    // were read at the end of the block before (or ahead of the loop)
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int l = s >> 2, j = s & 3;
      if (s < 7) lds_read(a[(s + 1) & 1], lds_lane, cur * (A4 * 16) + (((s + 1) & 3) * 4 + 2 * ((s + 1) >> 2)) * (ROWS * 16));
      lds_wait(a[s & 1], s < 7);
#pragma unroll
      for (int y = 0; y < NP; ++y) {
        const v4i b = expand_codes((uint32_t)wset[cur][y][l][j]);
#pragma unroll
        for (int rt2 = 0; rt2 < RT2W; ++rt2)
          acc[rt2][y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[s & 1][rt2], b, acc[rt2][y], 0, 0, 0);
      }
    }
    // blocks issued after kb+1 and still allowed in flight: kb+2 .. min(kb+NS-1, nb-1)
    wait_blocks(min(kb + NS - 1, nb - 1) - (kb + 1));
    tie_w(wset[n1]);
    __builtin_amdgcn_s_barrier();
    lds_read(a[0], lds_lane, n1 * (A4 * 16));  // after the last block: a read of stale rows, waited for below
  };
  lds_read(a[0], lds_lane, 0);
  int kb = 0;
  for (; kb + NS <= nb; kb += NS) {  // one exit only: the accumulators keep their registers
    block(std::integral_constant<int, 0>{}, kb);
    block(std::integral_constant<int, 1>{}, kb + 1);
    block(std::integral_constant<int, 2>{}, kb + 2);
    if constexpr (NS > 3) block(std::integral_constant<int, 3>{}, kb + 3);
  }
  if (kb < nb) {
    block(std::integral_constant<int, 0>{}, kb);
    if (kb + 1 < nb) block(std::integral_constant<int, 1>{}, kb + 1);
    if constexpr (NS > 3) {
      if (kb + 2 < nb) block(std::integral_constant<int, 2>{}, kb + 2);
    }
  }

  lds_wait(a[0], false);  // the read issued behind the last block
  unsigned tid_e = threadIdx.x;
  asm volatile("" : "+v"(tid_e));
  if constexpr (KSPLIT) {
    // Partial sums out, one coalesced KiB per register; the last workgroup of the tile to arrive adds
    // the others' to its own and goes on to the epilogue. Integer adds: the order does not matter.
    constexpr int NREG = RT2W * NP * 16;
    const int tile_id = bm * pr.grid_n + bn;
    int32_t *mine = pr.kpart + ((size_t)tile_id * ksn + ks) * (size_t)(NREG * TK_GEMM_THREADS) + tid_e;
#pragma unroll
    for (int rt2 = 0; rt2 < RT2W; ++rt2)
#pragma unroll
      for (int y = 0; y < NP; ++y)
#pragma unroll
        for (int c = 0; c < 16; ++c)
          __hip_atomic_store(mine + ((rt2 * NP + y) * 16 + c) * TK_GEMM_THREADS, acc[rt2][y][c], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    // Hand-off between workgroups without a fence. What it relies on, instruction by instruction (gfx950 follows
    // the gfx942 memory model of the LLVM AMDGPU backend):
    //  * every access to the partial sums and to the counter is an agent-scope atomic, i.e. carries sc1: such a
    //    store is written through the XCD's L2 to the memory side (where the XCDs' L2s meet), such a load never
    //    hits a line another XCD made stale, and the counter's read-modify-write executes at that same level;
    //  * vmcnt counts a store until it is acknowledged at the level its scope names, so `s_waitcnt vmcnt(0)` in
    //    EVERY thread followed by the workgroup barrier means all 256 threads' partial sums are visible device-wide
    //    before thread 0 issues the counter's increment -- the instruction pair a release at agent scope expands
    //    to, minus its `buffer_wbl2 sc1` write-back of the whole L2, which only earlier NON-sc1 stores would need
    //    (there are none whose values another workgroup reads);
    //  * the workgroup that reads ksn-1 from the counter is by construction the last to arrive; its loads of the
    //    others' sums are issued after the counter's value has come back (the value travels through LDS, a
    //    barrier and a branch, and a wave issues in order), and being sc1 loads they need no `buffer_inv sc1`,
    //    the other half of an acquire.
    // A device-scope fence per workgroup was measured at several times the kernel; the forced-slice tests cover
    // the result, tests/test_ksplit_protocol.py the counting protocol over every interleaving of arrivals.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int *arrived = (int *)smem;  // the A slots are free after the main loop's last barrier
    if (tid_e == 0) *arrived = __hip_atomic_fetch_add(pr.kcount + tile_id, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*arrived != ksn - 1) return;
    for (int k2 = 0; k2 < ksn; ++k2) {
      if (k2 == ks) continue;
      int32_t *theirs = pr.kpart + ((size_t)tile_id * ksn + k2) * (size_t)(NREG * TK_GEMM_THREADS) + tid_e;
#pragma unroll
      for (int rt2 = 0; rt2 < RT2W; ++rt2)
#pragma unroll
        for (int y = 0; y < NP; ++y)
#pragma unroll
          for (int c = 0; c < 16; ++c)
            acc[rt2][y][c] += __hip_atomic_load(theirs + ((rt2 * NP + y) * 16 + c) * TK_GEMM_THREADS, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
    }
    if (tid_e == 0) __hip_atomic_store(pr.kcount + tile_id, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero again for the next launch
    __syncthreads();  // `arrived` was read by everyone before the epilogue reuses the LDS
  }
  tk_gemm32_epilogue<P, NT, WR>(pr, hot, scales, acc, smem, (int)tid_e, bm, bn);
}

template <int P, int NT, int WR>
__device__ __forceinline__ void tk_gemm32_epilogue(const TkProblem &pr, const TkHot &hot, const float *const (&scales)[P],
                                                   v16i (&acc)[2 / WR][NT * P / 2], uint8_t *smem, int tid, int bm, int bn) {
  constexpr int ROWS = 64, A4 = 16 * ROWS, CST = TK_GEMM32_STAGES * A4 * 16, HP = NT / 2;
  constexpr int WC = TK_GEMM_WAVES / WR, RT2W = 2 / WR;
  const int wave = tid >> 6, lane = tid & 63, r16 = lane & 15, h = (lane >> 4) & 1, kappa = lane >> 5;
  const int wr = WR == 1 ? 0 : wave / WC, wc = WR == 1 ? wave : wave % WC;
  const int R = hot.R, row0 = bm * ROWS, tile0 = (bn * WC + wc) * NT;
  const int n_tiles = (hot.n + 15) >> 4;
  const int *cst_rs = (const int *)(smem + CST);
  const float *cst_as = (const float *)(smem + CST + 256);
  const int *cst_exp = (const int *)(smem + CST + 512);
  const int *cst_flag = (const int *)(smem + CST + 768);
  unsigned my_flag = 0;
  if (hot.flags && tid < ROWS) {
    const bool in_range = hot.mode == TK_MODE_INT8 ? row0 + tid < R : (row0 >> 2) + tid < hot.M;
    if (in_range) my_flag = cst_flag[tid] ? 1u : 0u;
  }
  // this lane's column in pair z of every plane: tile 2z + h, column r16
  float sc[HP][P];
#pragma unroll
  for (int z = 0; z < HP; ++z) {
    const int t = tile0 + 2 * z + h, n = t * 16 + r16;
#pragma unroll
    for (int p = 0; p < P; ++p) sc[z][p] = (t < n_tiles && n < hot.n) ? gload(scales[p] + n) : 0.0f;
  }
  const int wg_flag = __syncthreads_or((int)my_flag);
  // constants of the 4 rows rl..rl+3 of the tile (rl a multiple of 4)
  auto row_const = [&](int rl) {
    RowConst rc;
    const v4i rs4 = *(const v4i *)(cst_rs + rl);
    const float4 as4 = *(const float4 *)(cst_as + rl);
    rc.rs[0] = rs4.x; rc.rs[1] = rs4.y; rc.rs[2] = rs4.z; rc.rs[3] = rs4.w;
    rc.as[0] = as4.x; rc.as[1] = as4.y; rc.as[2] = as4.z; rc.as[3] = as4.w;
    rc.exp = cst_exp[rl >> 2];
    rc.flag = 0;
    if (wg_flag) {
      if (hot.mode == TK_MODE_INT8) {
        const v4i f4 = *(const v4i *)(cst_flag + rl);
        rc.flag = (f4.x ? 1u : 0u) | (f4.y ? 2u : 0u) | (f4.z ? 4u : 0u) | (f4.w ? 8u : 0u);
      } else {
        rc.flag = cst_flag[rl >> 2] ? 1u : 0u;
      }
    }
    return rc;
  };
  // the four accumulator registers 4q..4q+3 of row tile rt2, pair z, every plane
  auto quad = [&](int rt2, int q, int z, v4i (&av)[P]) {
#pragma unroll
    for (int p = 0; p < P; ++p) {
      const v16i &c = acc[rt2][p * HP + z];
      av[p] = v4i{c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]};
    }
  };

  const int esz = hot.out_dtype == TK_BF16 ? 2 : 4;
  // (a call with a fused residual add takes the direct stores: the residual is read where the value is formed)
  const bool staged = (((size_t)hot.n * esz) & 15) == 0 && (((size_t)hot.out) & 15) == 0 && !hot.residual;
  // The common case -- int8 contract, f32 or bf16 out, no row of the tile flagged -- as straight-line code
  // with compile-time strides: the general staging below decides contract, output type and flags per
  // output (about 25 instructions and several branches each, as long as a short K loop).
  auto lean = [&](auto esz_c, auto as_c) {
    constexpr int ESZ = decltype(esz_c)::value;
    constexpr bool HAS_AS = decltype(as_c)::value;
    constexpr int WG_COLS = WC * NT * 16, HALVES = ESZ == 4 ? 2 : 1, OROWS = 64 / HALVES;
    constexpr int STRIDE = WG_COLS * ESZ + 16, PIECES_ROW = WG_COLS * ESZ / 16, PER16 = 16 / ESZ;
    const int col0 = bn * WG_COLS;
    uint8_t *lane_base = smem + (size_t)(4 * kappa) * STRIDE + ((wc * NT + h) * 16 + r16) * ESZ;
    const int *lane_rs = cst_rs + 4 * kappa;
    const float *lane_as = cst_as + 4 * kappa;
#pragma unroll
    for (int hh = 0; hh < HALVES; ++hh) {
      if (hh > 0) __syncthreads();
#pragma unroll
      for (int rt2 = 0; rt2 < RT2W; ++rt2) {
        const int rtile = wr * RT2W + rt2;  // this wave's 32-row tile inside the 64 rows
        if (HALVES == 2 && rtile != hh) continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rl = rtile * 32 + 8 * q, sl = rl - (HALVES == 2 ? hh * 32 : 0);
          RowConst rc;
          const v4i rs4 = *(const v4i *)(lane_rs + rl);
          rc.rs[0] = rs4.x; rc.rs[1] = rs4.y; rc.rs[2] = rs4.z; rc.rs[3] = rs4.w;
          if (HAS_AS) {
            const float4 as4 = *(const float4 *)(lane_as + rl);
            rc.as[0] = as4.x; rc.as[1] = as4.y; rc.as[2] = as4.z; rc.as[3] = as4.w;
          }
#pragma unroll
          for (int z = 0; z < HP; ++z) {
            v4i av[P];
            quad(rt2, q, z, av);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float f = int8_value<P>(av, r, sc[z], rc, HAS_AS);
              uint8_t *dst = lane_base + (size_t)(sl + r) * STRIDE + z * 32 * ESZ;
              if (ESZ == 2) *(uint16_t *)dst = f32_to_bf16_hw(f); else *(float *)dst = f;
            }
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int it = 0; it < OROWS * PIECES_ROW / TK_GEMM_THREADS; ++it) {
        const int pc = it * TK_GEMM_THREADS + tid;
        const int rl = pc / PIECES_ROW, piece = pc % PIECES_ROW;
        const int orow = row0 + hh * OROWS + rl, c = col0 + piece * PER16;
        if (orow < R && c < hot.n)
          *(TK_GLOBAL v4u *)((uint8_t *)hot.out + ((size_t)orow * hot.n + c) * ESZ) = *(const v4u *)(smem + (size_t)rl * STRIDE + piece * 16);
      }
    }
  };
  if (staged && hot.mode == TK_MODE_INT8 && hot.out_dtype != TK_I32 && !wg_flag) {
    const bool has_as = hot.act_scale != nullptr;
    if (esz == 2) {
      if (has_as) lean(std::integral_constant<int, 2>{}, std::true_type{});
      else lean(std::integral_constant<int, 2>{}, std::false_type{});
    } else {
      if (has_as) lean(std::integral_constant<int, 4>{}, std::true_type{});
      else lean(std::integral_constant<int, 4>{}, std::false_type{});
    }
  } else if (staged) {
    constexpr int WG_COLS = WC * NT * 16;
    const bool int8_mode = hot.mode == TK_MODE_INT8 || hot.out_dtype == TK_I32;
    const int halves = esz == 4 ? 2 : 1;       // 4-byte outputs take the 64 rows in two halves
    const int orows_half = int8_mode ? (64 / halves) : (16 / halves);
    const int stride = WG_COLS * esz + 16;     // padded against bank conflicts
    const int pieces_row = WG_COLS * esz / 16;
    const int out_row0 = int8_mode ? row0 : (row0 >> 2);
    const int out_rows = int8_mode ? hot.R : hot.M;
    const int col0 = bn * WG_COLS;
    const bool has_as = hot.act_scale != nullptr;
    for (int hh = 0; hh < halves; ++hh) {
      if (hh > 0) __syncthreads();
#pragma unroll
      for (int rt2 = 0; rt2 < RT2W; ++rt2) {
        if (halves == 2 && wr * RT2W + rt2 != hh) continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rl = (wr * RT2W + rt2) * 32 + 8 * q + 4 * kappa;  // first of this lane's 4 rows, tile-local
          const int sl = rl - (halves == 2 ? hh * 32 : 0);         // ... staging-local
          const RowConst rc = row_const(rl);
#pragma unroll
          for (int z = 0; z < HP; ++z) {
            const int cl = (wc * NT + 2 * z + h) * 16 + r16;
            v4i av[P];
            quad(rt2, q, z, av);
            if (hot.out_dtype == TK_I32) {
#pragma unroll
              for (int r = 0; r < 4; ++r) *(int32_t *)(smem + (size_t)(sl + r) * stride + cl * 4) = av[0][r] - rc.rs[r];
            } else if (hot.mode == TK_MODE_INT8) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const float f = int8_value<P>(av, r, sc[z], rc, has_as);
                uint8_t *dst = smem + (size_t)(sl + r) * stride + cl * esz;
                if (esz == 2) *(uint16_t *)dst = f32_to_bf16_rne(f); else *(float *)dst = f;
              }
            } else {
              const float f = digits_value<P>(av, sc[z], rc);
              uint8_t *dst = smem + (size_t)(sl >> 2) * stride + cl * esz;
              if (esz == 2) *(uint16_t *)dst = f32_to_bf16_rne(f); else *(float *)dst = f;
            }
          }
        }
      }
      __syncthreads();
      const int per16 = 16 / esz;
      for (int pc = tid; pc < orows_half * pieces_row; pc += TK_GEMM_THREADS) {
        const int rl = pc / pieces_row, piece = pc - rl * pieces_row;
        const int orow = out_row0 + hh * orows_half + rl;
        const int c = col0 + piece * per16;
        if (orow >= out_rows || c >= hot.n) continue;
        if (wg_flag && hot.out_dtype != TK_I32 && gload(hot.flags + orow)) continue;  // written by exact_rows below
        *(TK_GLOBAL v4u *)((uint8_t *)hot.out + ((size_t)orow * hot.n + c) * esz) = *(const v4u *)(smem + (size_t)rl * stride + piece * 16);
      }
    }
  } else {
#pragma unroll
    for (int rt2 = 0; rt2 < RT2W; ++rt2)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int rl = (wr * RT2W + rt2) * 32 + 8 * q + 4 * kappa;
        const RowConst rc = row_const(rl);
#pragma unroll
        for (int z = 0; z < HP; ++z) {
          const int t = tile0 + 2 * z + h, n = t * 16 + r16;
          if (t >= n_tiles || n >= hot.n) continue;
          v4i av[P];
          quad(rt2, q, z, av);
          flow_epilogue<P>(hot, n, row0 + rl, av, sc[z], rc);
        }
      }
  }
  if (wg_flag) {
    for (int z = 0; z < HP; ++z) {
      const int t = tile0 + 2 * z + h, n = t * 16 + r16;
      if (t >= pr.n_tiles || n >= pr.n) continue;
      for (int rt2 = 0; rt2 < RT2W; ++rt2)
        for (int q = 0; q < 4; ++q) {
          const int rowbase = row0 + (wr * RT2W + rt2) * 32 + 8 * q + 4 * kappa;
          const unsigned fl = row_flags(pr, rowbase);
          if (fl) exact_rows(pr, n, rowbase, fl);
        }
    }
  }
}

// ------------------------------------------------------------------------------------------
// reference-order float kernel: one thread per (token, output)
// ------------------------------------------------------------------------------------------

__global__ __launch_bounds__(TK_WG) void tk_seq_kernel(TkProblem pr) {
  size_t idx = (size_t)blockIdx.x * TK_WG + threadIdx.x;
  size_t total = (size_t)pr.M * pr.n;
  if (idx >= total) return;
  int tok = (int)(idx / pr.n), n = (int)(idx % pr.n);
  float f = 0.0f;
  for (int p = 0; p < pr.planes; ++p) {
    float t = __fmul_rn(seq_dot(pr, p, n, tok, 0), pr.scales[p][n]);
    f = p == 0 ? t : __fadd_rn(f, t);
  }
  store_out(pr.out, pr.out_dtype, idx, f);
}

// ------------------------------------------------------------------------------------------
// upload-time re-layout
// ------------------------------------------------------------------------------------------

// TQ2_0 (66-byte blocks, only 2-byte aligned) -> T16. One thread per 16-byte piece.
// IEEE binary16 bits -> float, exact
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  const uint32_t sign = (h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
  if (exp == 0) return __uint_as_float(sign) + (sign ? -1.0f : 1.0f) * (float)man * 5.9604644775390625e-8f;  // man * 2^-24
  if (exp == 31) return __uint_as_float(sign | 0x7F800000u | (man << 13));
  return __uint_as_float(sign | ((exp + 112u) << 23) | (man << 13));
}

__global__ void tk_relayout_tq2_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ codes, size_t n,
                                       size_t nb, size_t pieces, int *invalid_row, float *__restrict__ block_scales) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= pieces) return;
  size_t l = idx & 63, chunk = idx >> 6;
  size_t kb = chunk % nb, t = chunk / nb;
  size_t row = t * 16 + (l & 15), g = l >> 4;
  uint32_t w[4] = {0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u};
  if (row < n) {
    const uint8_t *src = raw + (row * nb + kb) * 66 + g * 16;
    bool bad = false;
    for (int d = 0; d < 4; ++d) {
      uint32_t v = 0;
      for (int b = 0; b < 4; ++b) {
        uint32_t by = src[d * 4 + b];
        bad |= (by & (by >> 1) & 0x55u) != 0;  // reserved code 3 (crates/tritium-cpu/src/lib.rs:282-292)
        v |= by << (8 * b);
      }
      w[d] = v;
    }
    if (bad) atomicMin(invalid_row, (int)row);
  }
  ((uint4 *)codes)[idx] = make_uint4(w[0], w[1], w[2], w[3]);
  // the block's f16 scale (crates/tritium-format/src/lib.rs:359-371), kept for the block-scale planes:
  // entry (chunk, row of the tile) as f32, 0 for the padding rows of the last tile
  if (block_scales && g == 0) {
    float sc = 0.0f;
    if (row < n) {
      const uint8_t *blk = raw + (row * nb + kb) * 66;
      sc = f16_bits_to_f32((uint32_t)blk[64] | ((uint32_t)blk[65] << 8));
    }
    block_scales[chunk * 16 + (l & 15)] = sc;
  }
}

// TQ1_0 (54-byte base-3 blocks, crates/tritium-format/src/tq1.rs:85-121) -> T16 2-bit codes.
__global__ void tk_relayout_tq1_kernel(const uint8_t *__restrict__ raw, uint8_t *__restrict__ codes, size_t n,
                                       size_t nb, size_t pieces) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= pieces) return;
  size_t l = idx & 63, chunk = idx >> 6;
  size_t kb = chunk % nb, t = chunk / nb;
  size_t row = t * 16 + (l & 15), g = l >> 4;
  uint32_t w[4] = {0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u};
  if (row < n) {
    const uint8_t *blk = raw + (row * nb + kb) * 54;
    const uint32_t pow3[5] = {1, 3, 9, 27, 81};
    for (int d = 0; d < 4; ++d) {
      uint32_t v = 0;
      for (int b = 0; b < 4; ++b) {
        int byteidx = (int)g * 16 + d * 4 + b;
        int c = byteidx >> 5, mm = byteidx & 31;
        uint32_t by = 0;
        for (int s = 0; s < 4; ++s) {
          int e = c * 128 + s * 32 + mm;
          uint32_t src, dig;
          if (e < 160) { src = blk[e & 31]; dig = e >> 5; }
          else if (e < 240) { src = blk[32 + ((e - 160) & 15)]; dig = (e - 160) >> 4; }
          else { src = blk[48 + ((e - 240) & 3)]; dig = (e - 240) >> 2; }
          uint32_t q = (src * pow3[dig]) & 0xFFu;   // u8 wraparound is part of the scheme
          uint32_t code = (q * 3u) >> 8;            // {0,1,2} = trit + 1
          by |= code << (2 * s);
        }
        v |= by << (8 * b);
      }
      w[d] = v;
    }
  }
  ((uint4 *)codes)[idx] = make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ void tk_decode_trits_kernel(const uint8_t *__restrict__ codes, size_t n, size_t k, size_t nb,
                                       int8_t *__restrict__ trits) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n * k) return;
  int row = (int)(idx / k), kk = (int)(idx % k);
  trits[idx] = (int8_t)(code_at(codes, (int)nb, row, kk) - 1);
}

// ------------------------------------------------------------------------------------------
// activation prep: one workgroup per token
// ------------------------------------------------------------------------------------------

// Row maximum and "any lane saw NaN/Inf" in one pass through LDS (one barrier pair instead of two).
__device__ void block_max_any(float &v, int &flag, float *sh, int *shi) {
  for (int o = 32; o > 0; o >>= 1) {
    v = fmaxf(v, __shfl_xor(v, o));
    flag |= __shfl_xor(flag, o);
  }
  if ((threadIdx.x & 63) == 0) {
    sh[threadIdx.x >> 6] = v;
    shi[threadIdx.x >> 6] = flag;
  }
  __syncthreads();
  v = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
  flag = shi[0] | shi[1] | shi[2] | shi[3];
  __syncthreads();
}

// NV block sums at once (the four digit rows of a token, and its two element counts); sh holds
// 4 * NV ints.
template <int NV>
__device__ void block_sums(int (&v)[NV], int *sh) {
#pragma unroll
  for (int d = 0; d < NV; ++d)
    for (int o = 32; o > 0; o >>= 1) v[d] += __shfl_xor(v[d], o);
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int d = 0; d < NV; ++d) sh[(threadIdx.x >> 6) * NV + d] = v[d];
  }
  __syncthreads();
#pragma unroll
  for (int d = 0; d < NV; ++d) v[d] = sh[d] + sh[NV + d] + sh[2 * NV + d] + sh[3 * NV + d];
  __syncthreads();
}

__device__ int block_sum(int v, int *sh) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  int r = sh[0] + sh[1] + sh[2] + sh[3];
  __syncthreads();
  return r;
}

// Four consecutive activations starting at element e (a multiple of 4) as floats; elements at or
// past k read as 0. `vec` says the row starts are aligned for one 8- or 16-byte load.
__device__ __forceinline__ void load_act4(const void *act, int dtype, size_t base, size_t e, size_t k, bool vec, float (&v)[4]) {
  if (vec && e + 4 <= k) {
    if (dtype == TK_BF16) {
      typedef unsigned v2u __attribute__((ext_vector_type(2)));
      const v2u u = *(const TK_GLOBAL v2u *)((const uint16_t *)act + base + e);
      v[0] = __uint_as_float(u.x << 16);
      v[1] = __uint_as_float(u.x & 0xFFFF0000u);
      v[2] = __uint_as_float(u.y << 16);
      v[3] = __uint_as_float(u.y & 0xFFFF0000u);
    } else {
      const v4u u = *(const TK_GLOBAL v4u *)((const float *)act + base + e);
      v[0] = __uint_as_float(u.x);
      v[1] = __uint_as_float(u.y);
      v[2] = __uint_as_float(u.z);
      v[3] = __uint_as_float(u.w);
    }
    return;
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) v[b] = e + b < k ? load_act(act, dtype, base + e + b) : 0.0f;
}

__device__ __forceinline__ bool act_rows_vectorizable(const void *act, int dtype, size_t k) {
  return (k & 3) == 0 && (((size_t)act) & 15) == 0 && (dtype == TK_BF16 || dtype == TK_F32);
}

// gamma = max |a| with the reference's `a > gamma` rule (NaN never wins), plus a non-finite flag.
// RMSNorm in front of the quantization (crates/tritium-nn/src/ops/rmsnorm.rs:21-96). The sum of
// squares folds in the reference's canonical order: slot t (= thread t of the 256) takes x[t],
// x[t+256], ... in ascending order, multiply then add, and a power-of-two tree (off = 128 .. 1)
// combines the slots; then inv = 1 / sqrt(sum / k + eps), every operation rounded once.
struct RowNorm {
  int kind;        // 0 none, 1 scale w, 2 scale 1 + w
  float inv;
  const float *w;
};

__device__ float row_inv_rms(const void *act, int dtype, size_t base, size_t k, float eps, float *part /* [256] */) {
  static_assert(TK_WG == 256, "the canonical reduction has 256 slots");
  float acc = 0.0f;
  for (size_t i = threadIdx.x; i < k; i += 256) {
    const float v = load_act(act, dtype, base + i);
    acc = __fadd_rn(acc, __fmul_rn(v, v));
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) part[threadIdx.x] = __fadd_rn(part[threadIdx.x], part[threadIdx.x + off]);
    __syncthreads();
  }
  const float mean_sq = __fdiv_rn(part[0], (float)k);
  __syncthreads();
  // sqrtf, not __fsqrt_rn: without OCML_BASIC_ROUNDED_OPERATIONS the latter is the approximate
  // native square root; sqrtf and "/" are correctly rounded (hipcc's default for fp32)
  return __fdiv_rn(1.0f, sqrtf(__fadd_rn(mean_sq, eps)));
}

// y = (x * inv) * scale(w), left to right (rmsnorm.rs:91-93)
__device__ __forceinline__ void apply_norm4(const RowNorm &nm, size_t e, size_t k, float (&v)[4]) {
  if (!nm.kind) return;
  float w[4];
  if (e + 4 <= k && (((size_t)nm.w) & 15) == 0) {  // e is a multiple of 4
    const v4u u = *(const TK_GLOBAL v4u *)(nm.w + e);
    w[0] = __uint_as_float(u.x);
    w[1] = __uint_as_float(u.y);
    w[2] = __uint_as_float(u.z);
    w[3] = __uint_as_float(u.w);
  } else {
#pragma unroll
    for (int b = 0; b < 4; ++b) w[b] = e + b < k ? gload(nm.w + e + b) : 0.0f;
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    if (e + b >= k) continue;
    const float sc = nm.kind == 2 ? __fadd_rn(1.0f, w[b]) : w[b];
    v[b] = __fmul_rn(__fmul_rn(v[b], nm.inv), sc);
  }
}

__device__ void row_absmax(const void *act, int dtype, size_t base, size_t k, bool vec, float *sh, float &gamma,
                           int &nonfinite, int *shi, const RowNorm &nm = RowNorm{0, 0.0f, nullptr}) {
  float g = 0.0f;
  int nf = 0;
  for (size_t e = (size_t)threadIdx.x * 4; e < k; e += TK_WG * 4) {
    float v[4];
    load_act4(act, dtype, base, e, k, vec, v);
    apply_norm4(nm, e, k, v);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float a = fabsf(v[b]);
      if (a > g) g = a;
      nf |= !(a <= 3.402823466e38f);  // NaN or Inf
    }
  }
  block_max_any(g, nf, sh, shi);
  gamma = g;
  nonfinite = nf != 0;
}

// uniform_m > 0: every tensor of the table has that many tokens, so the entry follows from the
// workgroup index without the chain of dependent loads the search costs.
__device__ __forceinline__ const TkPrep &find_prep(const TkPrep &single, const TkPrep *table, int nprep, int uniform_m,
                                                   int &row) {
  if (!table) {
    // Workgroups go to the 8 XCDs in turn, and 8 consecutive rows share every 128-byte line of the
    // operand layout (16 bytes each). With the rows taken in this order a line is written by one XCD,
    // so its pieces meet in one L2 and leave it as a whole line, not as eight masked writes.
    const unsigned blk = blockIdx.x;
    if ((gridDim.x & 63u) == 0) {
      const unsigned xcd = blk & 7u, slot = blk >> 3;
      row = (int)((((slot >> 3) * 8u + xcd) * 8u) + (slot & 7u));
    } else {
      row = (int)blk;
    }
    return single;
  }
  if (uniform_m > 0) {
    const int t = (int)blockIdx.x / uniform_m;
    row = (int)blockIdx.x - t * uniform_m;
    return table[t];
  }
  int lo = 0, hi = nprep - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (table[mid].row_begin <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  row = blockIdx.x - table[lo].row_begin;
  return table[lo];
}

// The 16 elements of operand piece (kb, q16) of a row: four groups of four, 32 elements apart.
__device__ __forceinline__ void load_piece(const void *act, int dtype, size_t base, size_t e0, size_t k, bool vec,
                                           float (&v)[16]) {
#pragma unroll
  for (int sl = 0; sl < 4; ++sl) {
    float t[4];
    load_act4(act, dtype, base, e0 + (size_t)sl * 32, k, vec, t);
#pragma unroll
    for (int b = 0; b < 4; ++b) v[sl * 4 + b] = t[b];
  }
}

// Rows of up to TK_PREP_HELD * 256 pieces (K <= 16384) are read from memory once: every thread keeps
// its pieces in registers between the pass that finds the row maximum and the pass that quantizes.
#define TK_PREP_HELD 4
template <int HELD>
__device__ __forceinline__ void row_absmax_held(const void *act, int dtype, size_t base, size_t k, size_t npieces,
                                                bool vec, float (&held)[HELD][16], float *sh, float &gamma,
                                                int &nonfinite, int *shi) {
  float g = 0.0f;
  int nf = 0;
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)threadIdx.x + (size_t)it * TK_WG;
    if (pc < npieces) {
      load_piece(act, dtype, base, piece_elem0(pc >> 4, (int)(pc & 15)), k, vec, held[it]);
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const float a = fabsf(held[it][x]);  // elements past k were loaded as 0
        if (a > g) g = a;
        nf |= !(a <= 3.402823466e38f);
      }
    }
  }
  block_max_any(g, nf, sh, shi);
  gamma = g;
  nonfinite = nf != 0;
}

// Per-token int8 absmax quant (crates/tritium-spec/src/lib.rs:351-378) straight into operand order.
// HELD = pieces a thread keeps in registers: 1 for rows of up to 256 pieces (K <= 4096), 2 up to 512:
// the registers saved double the resident workgroups, so that 2048 tokens run as one round.
template <int HELD>
__global__ __launch_bounds__(TK_WG) void tk_prep_a8_kernel(TkPrep single, const TkPrep *__restrict__ table,
                                                           int nprep, int uniform_m) {
  __shared__ float shf[4];
  __shared__ int shi[4];
  int rowi;
  const TkPrep &pp = find_prep(single, table, nprep, uniform_m, rowi);
  const size_t row = rowi, k = pp.k, nb = pp.nb, R = pp.rs;
  const size_t base = row * k;
  const void *act = pp.act;
  const int dtype = pp.act_dtype;
  int8_t *ap = pp.ap, *qrm = pp.q_rowmajor;
  const bool vec = act_rows_vectorizable(act, dtype, k);
  RowNorm nm = {pp.norm_kind, 0.0f, pp.norm_w};
  float *ynorm = nullptr;
  if (nm.kind) {
    __shared__ float part[TK_WG];
    nm.inv = row_inv_rms(act, dtype, base, k, pp.norm_eps, part);
  }
  const size_t npieces = nb * 16;
  const bool resident = !nm.kind && npieces <= (size_t)HELD * TK_WG;
  float held[HELD][16];
  float gamma;
  int nonfinite;
  if (resident)
    row_absmax_held(act, dtype, base, k, npieces, vec, held, shf, gamma, nonfinite, shi);
  else
    row_absmax(act, dtype, base, k, vec, shf, gamma, nonfinite, shi, nm);
  if (nm.kind && nonfinite) ynorm = pp.ynorm;  // only the exact fallback reads the normalized row
  const float s = gamma == 0.0f ? 0.0f : __fdiv_rn(127.0f, gamma);  // one divide
  const bool live = gamma != 0.0f && !nonfinite;
  int sum = 0;
  // quantize the 16 values of piece pc and store them in operand order (and row-major, if asked)
  auto emit = [&](size_t pc, const float (&v)[16]) {
    const size_t kb = pc >> 4;
    const int q16 = (int)(pc & 15);
    const size_t e0 = piece_elem0(kb, q16);
    v4u piece;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const size_t e = e0 + (size_t)sl * 32;
      if (ynorm) {
#pragma unroll
        for (int b = 0; b < 4; ++b)
          if (e + b < k) gstore(ynorm + base + e + b, v[sl * 4 + b]);
      }
      uint32_t packed = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int q = 0;
        if (live && e + b < k) {
          float r = rintf(__fmul_rn(v[sl * 4 + b], s));  // one multiply, ties to even
          r = r < -128.0f ? -128.0f : (r > 127.0f ? 127.0f : r);
          q = (int)r;
        }
        sum += q;
        packed |= ((uint32_t)q & 0xFFu) << (8 * b);
      }
      piece[sl] = packed;
      if (qrm) {
        if (vec && e + 4 <= k) {
          *(TK_GLOBAL uint32_t *)(qrm + base + e) = packed;
        } else {
          for (int b = 0; b < 4; ++b)
            if (e + b < k) qrm[base + e + b] = (int8_t)(packed >> (8 * b));
        }
      }
    }
    if (ap) *(TK_GLOBAL v4u *)(ap + piece_offset(kb, q16, R, row)) = piece;
  };
  if (resident) {
#pragma unroll
    for (int it = 0; it < HELD; ++it) {
      const size_t pc = (size_t)threadIdx.x + (size_t)it * TK_WG;
      if (pc < npieces) emit(pc, held[it]);
    }
  } else {
    for (size_t pc = threadIdx.x; pc < npieces; pc += TK_WG) {
      float v[16];
      const size_t e0 = piece_elem0(pc >> 4, (int)(pc & 15));
      load_piece(act, dtype, base, e0, k, vec, v);
#pragma unroll
      for (int sl = 0; sl < 4; ++sl) {
        float t[4] = {v[sl * 4], v[sl * 4 + 1], v[sl * 4 + 2], v[sl * 4 + 3]};
        apply_norm4(nm, e0 + (size_t)sl * 32, k, t);
#pragma unroll
        for (int b = 0; b < 4; ++b) v[sl * 4 + b] = t[b];
      }
      emit(pc, v);
    }
  }
  sum = block_sum(sum, shi);
  if (threadIdx.x == 0) {
    if (pp.rowsum) pp.rowsum[row] = sum;
    pp.act_scale[row] = gamma == 0.0f ? 0.0f : __fdiv_rn(gamma, 127.0f);
    if (pp.aux) pp.aux[row] = s;
    if (pp.flags) pp.flags[row] = nonfinite ? 1u : 0u;
  }
}

// An element scaled onto the grid (r = a * 2^(30-E), q = its rounding) is carried faithfully when it
// lies on the grid or its rounding error is at most 2^-16 of it.
__device__ __forceinline__ bool digit_poor(float r, int q) { return !(fabsf(r) >= 32768.0f || r == (float)q); }

// Counts of the elements of one piece per magnitude band: band b holds 2^(30-4b-4) <= |r| < 2^(30-4b);
// elements below the eighth band (and zeros) are not counted.
__device__ __forceinline__ void count_bands(const float (&v)[16], int shift, int (&bands)[8]) {
#pragma unroll
  for (int x = 0; x < 16; ++x) {
    const float r = ldexpf(v[x], shift);
    const int band = (156 - (int)((__float_as_uint(r) >> 23) & 0xFFu)) >> 2;
#pragma unroll
    for (int b = 0; b < 8; ++b) bands[b] += band == b ? 1 : 0;
  }
}

#define TK_DIGITS_TRIM 96
// Energy left without the TK_DIGITS_TRIM largest elements, in units of 2^(2E): band b counts at its
// lower edge 2^(-4b-4). The grid does not carry the token when its rounding noise n_poor * 2^-62 / 3
// exceeds 2^-30 of that.
__device__ __forceinline__ bool digits_narrow(int n_poor, const int (&bands)[8]) {
  float left = 0.0f, edge2 = 0.00390625f;  // 2^-8
  int trim = TK_DIGITS_TRIM;
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const int c = bands[b], cut = c < trim ? c : trim;
    trim -= cut;
    left += (float)(c - cut) * edge2;
    edge2 *= 0.00390625f;
  }
  return n_poor > 0 && (float)n_poor > 3.0f * 4294967296.0f * left;
}

// Float token -> four balanced base-256 digit rows of round(a * 2^(30-E)), 2^(E-1) <= max|a| < 2^E.
// Scaling a float by a power of two is exact, so the rounding to an integer happens once, in
// single precision.
//
// Dynamic range. The grid is 2^(E-30) wide against the token's own maximum. An element that lies on
// the grid exactly, or is at least 2^(E-15) in magnitude (rounding error at most 2^-16 of itself), is
// carried faithfully; any other ("poor") element is rounded by up to 2^(E-31), which can be all of
// it. The reference's k-ordered f32 fold skips an activation under a zero trit
// (crates/tritium-core/src/reference.rs:42-51), so an output can miss the largest elements of a token
// and consist of small ones only: its value is then small next to the token's maximum, and the
// rounding of the poor elements shows. The prep therefore compares the rounding noise of a token,
// n_poor * 2^(2(E-31)) / 3, with the energy that is left when its TK_DIGITS_TRIM largest elements
// are all skipped (a lower bound from counts per 4-bit magnitude band below 2^E): where the noise
// exceeds 2^-30 of that energy (2^-15 in amplitude, i.e. 3e-5 of a typical output that misses the
// top elements), the token is flagged like one holding NaN or Inf and its outputs are computed in
// the reference's order. For every other token and every output, unconditionally,
//   |value - exact dot product| <= n * 2^(E-31)  (+ 1.5 ulp),  n = poor elements under its non-zero trits.
__global__ __launch_bounds__(TK_WG) void tk_prep_digits_kernel(TkPrep single, const TkPrep *__restrict__ table,
                                                               int nprep, int uniform_m) {
  __shared__ float shf[4];
  __shared__ int shi[32];
  int rowi;
  const TkPrep &pp = find_prep(single, table, nprep, uniform_m, rowi);
  const size_t tok = rowi, k = pp.k, nb = pp.nb, R = pp.rs;
  const size_t base = tok * k;
  const void *act = pp.act;
  const int dtype = pp.act_dtype;
  int8_t *ap = pp.ap;
  const bool vec = act_rows_vectorizable(act, dtype, k);
  const size_t npieces = nb * 16;
  const bool resident = npieces <= (size_t)TK_PREP_HELD * TK_WG;
  float held[TK_PREP_HELD][16];
  float gamma;
  int nonfinite;
  if (resident)
    row_absmax_held(act, dtype, base, k, npieces, vec, held, shf, gamma, nonfinite, shi);
  else
    row_absmax(act, dtype, base, k, vec, shf, gamma, nonfinite, shi);
  int E = 0;
  if (gamma != 0.0f && !nonfinite) (void)frexpf(gamma, &E);
  const int shift = 30 - E;
  const bool live = gamma != 0.0f && !nonfinite;
  int sums[5] = {0, 0, 0, 0, 0};  // four digit-row sums, poor elements
  int &n_poor = sums[4];
  // split the 16 values of piece pc into their four digit rows and store those in operand order
  auto emit = [&](size_t pc, const float (&v)[16]) {
    const size_t kb = pc >> 4;
    const int q16 = (int)(pc & 15);
    const size_t e0 = piece_elem0(kb, q16);
    v4u piece[4];
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const size_t e = e0 + (size_t)sl * 32;
      uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int q = 0;
        if (live && e + b < k) {
          const float r = ldexpf(v[sl * 4 + b], shift);
          q = __float2int_rn(r);  // |q| <= 2^30
          n_poor += digit_poor(r, q) ? 1 : 0;
        }
#pragma unroll
        for (int dg = 0; dg < 4; ++dg) {
          int dv = dg == 3 ? q : (((q + 128) & 0xFF) - 128);  // balanced digit in [-128,127]
          q = (q - dv) >> 8;
          sums[dg] += dv;
          packed[dg] |= ((uint32_t)dv & 0xFFu) << (8 * b);
        }
      }
#pragma unroll
      for (int dg = 0; dg < 4; ++dg) piece[dg][sl] = packed[dg];
    }
#pragma unroll
    for (int dg = 0; dg < 4; ++dg) *(TK_GLOBAL v4u *)(ap + piece_offset(kb, q16, R, tok * 4 + dg)) = piece[dg];
    if (pp.blocksum) {
      // sums of each digit row over this K block alone (the 16 pieces of a block sit in 16
      // consecutive lanes): entry [kb][row], row stride = the operand row count
      int bs[4];
#pragma unroll
      for (int dg = 0; dg < 4; ++dg) {
        int t = 0;
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
          const uint32_t u = piece[dg][sl];
          t += (int)(int8_t)(u & 0xFF) + (int)(int8_t)((u >> 8) & 0xFF) + (int)(int8_t)((u >> 16) & 0xFF) + (int)(int8_t)(u >> 24);
        }
        for (int o = 8; o > 0; o >>= 1) t += __shfl_xor(t, o);
        bs[dg] = t;
      }
      if (q16 == 0) {
#pragma unroll
        for (int dg = 0; dg < 4; ++dg) pp.blocksum[kb * pp.R + tok * 4 + dg] = bs[dg];
      }
    }
  };
  if (resident) {
#pragma unroll
    for (int it = 0; it < TK_PREP_HELD; ++it) {
      const size_t pc = (size_t)threadIdx.x + (size_t)it * TK_WG;
      if (pc < npieces) emit(pc, held[it]);
    }
  } else {
    for (size_t pc = threadIdx.x; pc < npieces; pc += TK_WG) {
      float v[16];
      load_piece(act, dtype, base, piece_elem0(pc >> 4, (int)(pc & 15)), k, vec, v);
      emit(pc, v);
    }
  }
  block_sums<5>(sums, shi);
  // Only a token that has poor elements needs the magnitude bands (the same answer in every thread, so
  // the barriers inside are reached by all or by none).
  bool narrow = false;
  if (sums[4] > 0) {
    int bands[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (resident) {
#pragma unroll
      for (int it = 0; it < TK_PREP_HELD; ++it) {
        const size_t pc = (size_t)threadIdx.x + (size_t)it * TK_WG;
        if (pc < npieces) count_bands(held[it], shift, bands);
      }
    } else {
      for (size_t pc = threadIdx.x; pc < npieces; pc += TK_WG) {
        float v[16];
        load_piece(act, dtype, base, piece_elem0(pc >> 4, (int)(pc & 15)), k, vec, v);
        count_bands(v, shift, bands);
      }
    }
    block_sums<8>(bands, shi);
    narrow = digits_narrow(sums[4], bands);
  }
  if (threadIdx.x < 4) {
    const int t = threadIdx.x;
    pp.rowsum[tok * 4 + t] = t == 0 ? sums[0] : t == 1 ? sums[1] : t == 2 ? sums[2] : sums[3];
  }
  if (threadIdx.x == 0) {
    pp.exps[tok] = -shift;
    pp.flags[tok] = (nonfinite || narrow) ? 1u : 0u;
  }
}

// ------------------------------------------------------------------------------------------
// activation prep, one WAVE per token: rows of up to HELD * 64 pieces (K <= 4096 at HELD = 4). Same
// arithmetic and the same bytes out as the one-workgroup-per-token kernels above; what changes is the
// shape of the work: a token's pieces sit in the registers of one wave, the row maximum and the row
// sums are wave shuffles, nothing waits at a barrier, every lane has pieces to work on (a K = 2048
// row has 128 pieces: half a workgroup's threads idle), and a launch has a quarter of the workgroups.
// Not for rows that are normalized first (the canonical sum of squares has 256 slots) nor for the
// per-block row sums of the block-scale planes.
// ------------------------------------------------------------------------------------------

// The token a wave works on, and its tensor. Single tensor, workgroup count a multiple of 16: eight
// consecutive rows share every 128-byte line of the operand layout, and workgroups go to the 8 XCDs
// in turn, so the two workgroups that cover rows 8j..8j+7 are taken from the same XCD.
// (team: the threads working on one token -- a wave, or the whole workgroup)
__device__ __forceinline__ const TkPrep &find_prep_wave(const TkPrep &single, const TkPrep *table, int nprep,
                                                        int uniform_m, int wave, int &row, int &gt, int team = 64) {
  const unsigned blk = blockIdx.x;
  if (team != 64) {
    gt = (int)blk;
    if (!table) {
      // Eight consecutive tokens share every 128-byte line of the operand rows (16 bytes each): workgroups
      // id, id + 8, ... run on one XCD, so give that XCD runs of eight tokens and its L2 whole lines to
      // write back.
      if ((gridDim.x & 63u) == 0) {
        const unsigned xcd = blk & 7u, slot = blk >> 3;
        gt = (int)((((slot >> 3) * 8u + xcd) * 8u) + (slot & 7u));
      }
      row = gt;
      return single;
    }
    if (uniform_m > 0) {
      const int t = min(gt / uniform_m, nprep - 1);
      row = gt - t * uniform_m;
      return table[t];
    }
    int lo = 0, hi = nprep - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (table[mid].row_begin <= gt) lo = mid; else hi = mid - 1;
    }
    row = gt - table[lo].row_begin;
    return table[lo];
  }
  if (!table) {
    if ((gridDim.x & 15u) == 0) {
      const unsigned xcd = blk & 7u, slot = blk >> 3;
      gt = (int)((((slot >> 1) * 8u + xcd) * 8u) + (slot & 1u) * 4u) + wave;
    } else {
      gt = (int)blk * 4 + wave;
    }
    row = gt;
    return single;
  }
  gt = (int)blk * 4 + wave;
  if (uniform_m > 0) {
    const int t = min(gt / uniform_m, nprep - 1);
    row = gt - t * uniform_m;
    return table[t];
  }
  int lo = 0, hi = nprep - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (table[mid].row_begin <= gt) lo = mid; else hi = mid - 1;
  }
  row = gt - table[lo].row_begin;
  return table[lo];
}

// FAST != 0: the launch's rows are whole K blocks (k a multiple of 256), 16-byte aligned, of one element type
// (1 = f32, 2 = bf16) and only the operand rows are wanted: no bound, alignment or type is tested per
// element, which is most of what the general form executes (a wave works through its token alone, one
// dependent instruction after the other: the instruction count is the launch's time).
template <int HELD, int FAST = 0, int TEAM = 64>
__device__ __forceinline__ void wave_absmax_held(const void *act, int dtype, size_t base, size_t k, size_t npieces, bool vec,
                                                 int lane, float (&held)[HELD][16], float &gamma, int &nonfinite,
                                                 float *shf = nullptr, int *shi = nullptr) {
  float g = 0.0f;
  int nf = 0;
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * TEAM;
    if (pc < npieces) {
      if constexpr (FAST != 0) load_piece_fast<FAST>(act, base, piece_elem0(pc >> 4, (int)(pc & 15)), held[it]);
      else load_piece(act, dtype, base, piece_elem0(pc >> 4, (int)(pc & 15)), k, vec, held[it]);
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const float a = fabsf(held[it][x]);  // elements past k were loaded as 0
        if (a > g) g = a;                    // NaN never wins (crates/tritium-spec/src/lib.rs:351-360)
        nf |= !(a <= 3.402823466e38f);
      }
    }
  }
  if constexpr (TEAM == 64) {
    for (int o = 32; o > 0; o >>= 1) {
      g = fmaxf(g, __shfl_xor(g, o));
      nf |= __shfl_xor(nf, o);
    }
  } else {
    block_max_any(g, nf, shf, shi);
  }
  gamma = g;
  nonfinite = nf != 0;
}

// TEAM = 64: a wave per token, four tokens per workgroup, no barrier. TEAM = 256: the workgroup per token (the
// maximum and the sums cross its waves through LDS): a quarter of the instructions per thread, for launches
// of few tokens, whose time is one token's chain.
template <int HELD, int FAST = 0, int TEAM = 64>
__global__ __launch_bounds__(TK_WG) void tk_prep_a8_wave_kernel(TkPrep single, const TkPrep *__restrict__ table, int nprep,
                                                                int uniform_m, unsigned rows) {
  __shared__ float shf[4];
  __shared__ int shi[4];
  const int wave = threadIdx.x >> 6, lane = TEAM == 64 ? (threadIdx.x & 63) : threadIdx.x;
  int rowi, gt;
  const TkPrep &pp = find_prep_wave(single, table, nprep, uniform_m, wave, rowi, gt, TEAM);
  if ((unsigned)gt >= rows) return;  // (a whole team leaves together: the barriers below stay uniform)
  const size_t row = rowi, k = pp.k, nb = pp.nb, R = pp.rs;
  const size_t base = row * k;
  const void *act = pp.act;
  const int dtype = pp.act_dtype;
  int8_t *ap = pp.ap, *qrm = pp.q_rowmajor;
  const bool vec = act_rows_vectorizable(act, dtype, k);
  const size_t npieces = nb * 16;
  float held[HELD][16];
  float gamma;
  int nonfinite;
  wave_absmax_held<HELD, FAST, TEAM>(act, dtype, base, k, npieces, vec, lane, held, gamma, nonfinite, shf, shi);
  const float s = gamma == 0.0f ? 0.0f : __fdiv_rn(127.0f, gamma);  // one divide
  const bool live = gamma != 0.0f && !nonfinite;
  int sum = 0;
  if constexpr (FAST != 0) {
    // a multiply by 0 stands in for the tests of `live` (a row without a finite maximum quantizes to zeros)
    const float sl_ = live ? s : 0.0f;
#pragma unroll
    for (int it = 0; it < HELD; ++it) {
      const size_t pc = (size_t)lane + (size_t)it * TEAM;
      if (pc >= npieces) continue;
      v4u piece;
#pragma unroll
      for (int sl = 0; sl < 4; ++sl) {
        uint32_t packed = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          float x = held[it][sl * 4 + b];
          if (!live) x = 0.0f;  // (a NaN or Inf times zero would not be zero)
          float r = rintf(__fmul_rn(x, sl_));  // one multiply, ties to even
          r = __builtin_fminf(__builtin_fmaxf(r, -128.0f), 127.0f);
          const int q = (int)r;
          sum += q;
          packed |= ((uint32_t)q & 0xFFu) << (8 * b);
        }
        piece[sl] = packed;
      }
      *(TK_GLOBAL v4u *)(ap + piece_offset(pc >> 4, (int)(pc & 15), R, row)) = piece;
    }
  } else
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * TEAM;
    if (pc >= npieces) continue;
    const size_t kb = pc >> 4;
    const int q16 = (int)(pc & 15);
    const size_t e0 = piece_elem0(kb, q16);
    v4u piece;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const size_t e = e0 + (size_t)sl * 32;
      uint32_t packed = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int q = 0;
        if (live && e + b < k) {
          float r = rintf(__fmul_rn(held[it][sl * 4 + b], s));  // one multiply, ties to even
          r = r < -128.0f ? -128.0f : (r > 127.0f ? 127.0f : r);
          q = (int)r;
        }
        sum += q;
        packed |= ((uint32_t)q & 0xFFu) << (8 * b);
      }
      piece[sl] = packed;
      if (qrm) {
        if (vec && e + 4 <= k) {
          *(TK_GLOBAL uint32_t *)(qrm + base + e) = packed;
        } else {
          for (int b = 0; b < 4; ++b)
            if (e + b < k) qrm[base + e + b] = (int8_t)(packed >> (8 * b));
        }
      }
    }
    if (ap) *(TK_GLOBAL v4u *)(ap + piece_offset(kb, q16, R, row)) = piece;
  }
  if constexpr (TEAM == 64) sum = wave_sum(sum);
  else sum = block_sum(sum, shi);
  if (lane == 0) {
    if (pp.rowsum) pp.rowsum[row] = sum;
    pp.act_scale[row] = gamma == 0.0f ? 0.0f : __fdiv_rn(gamma, 127.0f);
    if (pp.aux) pp.aux[row] = s;
    if (pp.flags) pp.flags[row] = nonfinite ? 1u : 0u;
  }
}

template <int HELD, int FAST = 0, int TEAM = 64>
__global__ __launch_bounds__(TK_WG) void tk_prep_digits_wave_kernel(TkPrep single, const TkPrep *__restrict__ table,
                                                                    int nprep, int uniform_m, unsigned rows) {
  __shared__ float shf[4];
  __shared__ int shi[32];
  const int wave = threadIdx.x >> 6, lane = TEAM == 64 ? (threadIdx.x & 63) : threadIdx.x;
  int rowi, gt;
  const TkPrep &pp = find_prep_wave(single, table, nprep, uniform_m, wave, rowi, gt, TEAM);
  if ((unsigned)gt >= rows) return;
  const size_t tok = rowi, k = pp.k, nb = pp.nb, R = pp.rs;
  const size_t base = tok * k;
  const void *act = pp.act;
  const int dtype = pp.act_dtype;
  int8_t *ap = pp.ap;
  const bool vec = act_rows_vectorizable(act, dtype, k);
  const size_t npieces = nb * 16;
  float held[HELD][16];
  float gamma;
  int nonfinite;
  wave_absmax_held<HELD, FAST, TEAM>(act, dtype, base, k, npieces, vec, lane, held, gamma, nonfinite, shf, shi);
  int E = 0;
  if (gamma != 0.0f && !nonfinite) (void)frexpf(gamma, &E);
  const int shift = 30 - E;
  const bool live = gamma != 0.0f && !nonfinite;
  int sums[4] = {0, 0, 0, 0}, n_poor = 0;
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * TEAM;
    if (pc >= npieces) continue;
    const size_t kb = pc >> 4;
    const int q16 = (int)(pc & 15);
    const size_t e0 = piece_elem0(kb, q16);
    v4u piece[4];
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const size_t e = e0 + (size_t)sl * 32;
      uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int q = 0;
        if constexpr (FAST != 0) {  // every element is inside the row; a row without a finite maximum splits zeros
          const float r = ldexpf(live ? held[it][sl * 4 + b] : 0.0f, shift);
          q = __float2int_rn(r);  // |q| <= 2^30
          n_poor += digit_poor(r, q) ? 1 : 0;
        } else if (live && e + b < k) {
          const float r = ldexpf(held[it][sl * 4 + b], shift);
          q = __float2int_rn(r);  // |q| <= 2^30
          n_poor += digit_poor(r, q) ? 1 : 0;
        }
#pragma unroll
        for (int dg = 0; dg < 4; ++dg) {
          int dv = dg == 3 ? q : (((q + 128) & 0xFF) - 128);  // balanced digit in [-128,127]
          q = (q - dv) >> 8;
          sums[dg] += dv;
          packed[dg] |= ((uint32_t)dv & 0xFFu) << (8 * b);
        }
      }
#pragma unroll
      for (int dg = 0; dg < 4; ++dg) piece[dg][sl] = packed[dg];
    }
#pragma unroll
    for (int dg = 0; dg < 4; ++dg) *(TK_GLOBAL v4u *)(ap + piece_offset(kb, q16, R, tok * 4 + dg)) = piece[dg];
  }
  if constexpr (TEAM == 64) {
#pragma unroll
    for (int dg = 0; dg < 4; ++dg) sums[dg] = wave_sum(sums[dg]);
    n_poor = wave_sum(n_poor);
  } else {
    int five[5] = {sums[0], sums[1], sums[2], sums[3], n_poor};
    block_sums<5>(five, shi);
#pragma unroll
    for (int dg = 0; dg < 4; ++dg) sums[dg] = five[dg];
    n_poor = five[4];
  }
  bool narrow = false;
  if (n_poor > 0) {  // uniform over the team
    int bands[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int it = 0; it < HELD; ++it) {
      const size_t pc = (size_t)lane + (size_t)it * TEAM;
      if (pc < npieces) count_bands(held[it], shift, bands);
    }
    if constexpr (TEAM == 64) {
#pragma unroll
      for (int b = 0; b < 8; ++b) bands[b] = wave_sum(bands[b]);
    } else {
      block_sums<8>(bands, shi);
    }
    narrow = digits_narrow(n_poor, bands);
  }
  if (lane < 4) pp.rowsum[tok * 4 + lane] = lane == 0 ? sums[0] : lane == 1 ? sums[1] : lane == 2 ? sums[2] : sums[3];
  if (lane == 0) {
    pp.exps[tok] = -shift;
    pp.flags[tok] = (nonfinite || narrow) ? 1u : 0u;
  }
}

// y = RMSNorm(x) in place for the pieces of one token that the 256 threads hold (thread t: pieces t, t + 256, ...),
// through xs [k] and part [256] floats of LDS; see tk_prep_a8_norm_kernel. Every thread passes every barrier, and
// xs and part are free again on return.
template <int HELD>
__device__ __forceinline__ void norm_held_pieces(float (&held)[HELD][16], const float *norm_w, int norm_kind, float eps,
                                                 size_t k, size_t npieces, float *xs, float *part) {
  const int tid = threadIdx.x;
  float w[HELD][16];
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)tid + (size_t)it * TK_WG;
    if (pc >= npieces) continue;
    const size_t e0 = piece_elem0(pc >> 4, (int)(pc & 15));
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const v4u u = *(const TK_GLOBAL v4u *)(norm_w + e0 + (size_t)sl * 32);
      w[it][sl * 4 + 0] = __uint_as_float(u.x);
      w[it][sl * 4 + 1] = __uint_as_float(u.y);
      w[it][sl * 4 + 2] = __uint_as_float(u.z);
      w[it][sl * 4 + 3] = __uint_as_float(u.w);
      *(float4 *)(xs + e0 + (size_t)sl * 32) =
          make_float4(held[it][sl * 4], held[it][sl * 4 + 1], held[it][sl * 4 + 2], held[it][sl * 4 + 3]);
    }
  }
  __syncthreads();
  float acc = 0.0f;
  for (size_t i = tid; i < k; i += TK_WG) {
    const float v = xs[i];
    acc = __fadd_rn(acc, __fmul_rn(v, v));
  }
  part[tid] = acc;
  __syncthreads();
  if (tid < 128) part[tid] = __fadd_rn(part[tid], part[tid + 128]);
  __syncthreads();
  if (tid < 64) {
    float p = __fadd_rn(part[tid], part[tid + 64]);
    for (int off = 32; off > 0; off >>= 1) p = __fadd_rn(p, __shfl_down(p, off));  // lanes >= off hold values no one reads
    if (tid == 0) part[0] = p;  // (only this lane read part[0])
  }
  __syncthreads();
  const float mean_sq = __fdiv_rn(part[0], (float)k);
  __syncthreads();
  const float inv = __fdiv_rn(1.0f, sqrtf(__fadd_rn(mean_sq, eps)));  // (see row_inv_rms on sqrtf)
#pragma unroll
  for (int it = 0; it < HELD; ++it)
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      const float sc = norm_kind == 2 ? __fadd_rn(1.0f, w[it][x]) : w[it][x];
      held[it][x] = __fmul_rn(__fmul_rn(held[it][x], inv), sc);  // y = (x * inv) * scale(w), left to right
    }
}

// RMSNorm + quantization of rows of whole K blocks (16-byte aligned f32 or bf16 rows and norm weights, at most
// HELD pieces per thread, operand rows only) in one pass over memory: the token's pieces and their norm weights are
// loaded once and stay in registers. The sum of squares has to fold in the canonical order (slot t of 256 takes
// x[t], x[t+256], ... ascending, then the power-of-two tree; see row_inv_rms), which is not the order the pieces
// are held in, so the values cross LDS once in element order; the tree's levels below 64 pair lanes of the first
// wave exactly as the slots pair (slot t with slot t + off), by shuffles. Same bits as tk_prep_a8_kernel, which
// reads the row three times and crosses nine barriers for the tree alone. Entries without a norm skip that part.
template <int HELD, int FAST>
__global__ __launch_bounds__(TK_WG) void tk_prep_a8_norm_kernel(TkPrep single, const TkPrep *__restrict__ table,
                                                                int nprep, int uniform_m) {
  static_assert(TK_WG == 256, "the canonical reduction has 256 slots");
  __shared__ __attribute__((aligned(16))) float xs[HELD * 256 * 16];
  __shared__ float part[TK_WG];
  __shared__ float shf[4];
  __shared__ int shi[4];
  int rowi;
  const TkPrep &pp = find_prep(single, table, nprep, uniform_m, rowi);
  const size_t row = rowi, k = pp.k, nb = pp.nb, R = pp.rs;
  const size_t base = row * k, npieces = nb * 16;
  const int tid = threadIdx.x;
  float held[HELD][16];
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)tid + (size_t)it * TK_WG;
    if (pc < npieces) load_piece_fast<FAST>(pp.act, base, piece_elem0(pc >> 4, (int)(pc & 15)), held[it]);
  }
  if (pp.norm_kind) norm_held_pieces<HELD>(held, pp.norm_w, pp.norm_kind, pp.norm_eps, k, npieces, xs, part);  // uniform over the workgroup
  float g = 0.0f;
  int nf = 0;
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)tid + (size_t)it * TK_WG;
    if (pc >= npieces) continue;
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      const float a = fabsf(held[it][x]);
      if (a > g) g = a;  // NaN never wins (crates/tritium-spec/src/lib.rs:351-360)
      nf |= !(a <= 3.402823466e38f);
    }
  }
  block_max_any(g, nf, shf, shi);
  const float gamma = g;
  const bool nonfinite = nf != 0;
  const float s = gamma == 0.0f ? 0.0f : __fdiv_rn(127.0f, gamma);  // one divide
  const bool live = gamma != 0.0f && !nonfinite;
  const float sl_ = live ? s : 0.0f;
  float *ynorm = (pp.norm_kind && nonfinite) ? pp.ynorm : nullptr;  // only the exact fallback reads the normalized row
  int sum = 0;
#pragma unroll
  for (int it = 0; it < HELD; ++it) {
    const size_t pc = (size_t)tid + (size_t)it * TK_WG;
    if (pc >= npieces) continue;
    const size_t e0 = piece_elem0(pc >> 4, (int)(pc & 15));
    v4u piece;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      if (ynorm) {
#pragma unroll
        for (int b = 0; b < 4; ++b) gstore(ynorm + base + e0 + (size_t)sl * 32 + b, held[it][sl * 4 + b]);
      }
      uint32_t packed = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float x = held[it][sl * 4 + b];
        if (!live) x = 0.0f;  // (a NaN or Inf times zero would not be zero)
        float r = rintf(__fmul_rn(x, sl_));  // one multiply, ties to even
        r = __builtin_fminf(__builtin_fmaxf(r, -128.0f), 127.0f);
        const int q = (int)r;
        sum += q;
        packed |= ((uint32_t)q & 0xFFu) << (8 * b);
      }
      piece[sl] = packed;
    }
    *(TK_GLOBAL v4u *)(pp.ap + piece_offset(pc >> 4, (int)(pc & 15), R, row)) = piece;
  }
  sum = block_sum(sum, shi);
  if (tid == 0) {
    if (pp.rowsum) pp.rowsum[row] = sum;
    pp.act_scale[row] = gamma == 0.0f ? 0.0f : __fdiv_rn(gamma, 127.0f);
    if (pp.aux) pp.aux[row] = s;
    if (pp.flags) pp.flags[row] = nonfinite ? 1u : 0u;
  }
}

// ------------------------------------------------------------------------------------------
// Decode in one launch: the flow kernel builds the operand rows of its one to four tokens itself. Every workgroup
// repeats the prep kernels' work for all tokens -- a few elements per thread -- in place of a second launch in
// front of every call, which costs more than the kernel itself on a single layer. The arithmetic is that of
// tk_prep_a8_wave_kernel / tk_prep_digits_wave_kernel in their straight-line form with the workgroup as the team
// (whole K blocks, 16-byte aligned rows of f32 or bf16, at most two pieces per thread of the 256), statement for
// statement, so rows, row sums, scales, exponents and flags carry the same bits. They go to LDS: the rows in
// operand order at `rows`, the constants at `cst` (int rowsum[64] | float scale or int exponent [64] |
// uint flag[64] | float 127/gamma [64]).
// ------------------------------------------------------------------------------------------
// The tokens are taken one after the other (a version with the loads and reductions of four tokens at once was
// slower for one token and no faster for four: the kernel's code grows fourfold, and what a token costs is its
// arithmetic, about 25 instructions per element under the float contract, repeated by every workgroup).
#define TK_FUSED_HELD 2
template <int FAST>
__device__ __forceinline__ void fused_token_a8(const void *act, int tok, size_t k, size_t nb, size_t R, uint4 *rows,
                                               uint8_t *cst, float *shf, int *shi) {
  const int lane = threadIdx.x;
  const size_t npieces = nb * 16, base = (size_t)tok * k;
  float held[TK_FUSED_HELD][16];
  float gamma;
  int nonfinite;
  wave_absmax_held<TK_FUSED_HELD, FAST, 256>(act, 0, base, k, npieces, true, lane, held, gamma, nonfinite, shf, shi);
  const float s = gamma == 0.0f ? 0.0f : __fdiv_rn(127.0f, gamma);  // one divide
  const bool live = gamma != 0.0f && !nonfinite;
  const float sl_ = live ? s : 0.0f;
  int sum = 0;
#pragma unroll
  for (int it = 0; it < TK_FUSED_HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * 256;
    if (pc >= npieces) continue;
    uint4 piece;
    uint32_t *pw = (uint32_t *)&piece;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      uint32_t packed = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float x = held[it][sl * 4 + b];
        if (!live) x = 0.0f;  // (a NaN or Inf times zero would not be zero)
        float r = rintf(__fmul_rn(x, sl_));  // one multiply, ties to even
        r = __builtin_fminf(__builtin_fmaxf(r, -128.0f), 127.0f);
        const int q = (int)r;
        sum += q;
        packed |= ((uint32_t)q & 0xFFu) << (8 * b);
      }
      pw[sl] = packed;
    }
    rows[piece_offset(pc >> 4, (int)(pc & 15), R, (size_t)tok) >> 4] = piece;
  }
  sum = block_sum(sum, shi);
  if (lane == 0) {
    ((int *)cst)[tok] = sum;
    ((float *)(cst + 256))[tok] = gamma == 0.0f ? 0.0f : __fdiv_rn(gamma, 127.0f);
    ((uint32_t *)(cst + 512))[tok] = nonfinite ? 1u : 0u;
    ((float *)(cst + 768))[tok] = s;
  }
}

template <int FAST>
__device__ __forceinline__ void fused_token_digits(const void *act, int tok, size_t k, size_t nb, size_t R, uint4 *rows,
                                                   uint8_t *cst, float *shf, int *shi) {
  const int lane = threadIdx.x;
  const size_t npieces = nb * 16, base = (size_t)tok * k;
  float held[TK_FUSED_HELD][16];
  float gamma;
  int nonfinite;
  wave_absmax_held<TK_FUSED_HELD, FAST, 256>(act, 0, base, k, npieces, true, lane, held, gamma, nonfinite, shf, shi);
  int E = 0;
  if (gamma != 0.0f && !nonfinite) (void)frexpf(gamma, &E);
  const int shift = 30 - E;
  const bool live = gamma != 0.0f && !nonfinite;
  int five[5] = {0, 0, 0, 0, 0};  // four digit-row sums, poor elements
#pragma unroll
  for (int it = 0; it < TK_FUSED_HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * 256;
    if (pc >= npieces) continue;
    uint4 piece[4];
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float r = ldexpf(live ? held[it][sl * 4 + b] : 0.0f, shift);
        int q = __float2int_rn(r);  // |q| <= 2^30
        five[4] += digit_poor(r, q) ? 1 : 0;
#pragma unroll
        for (int dg = 0; dg < 4; ++dg) {
          int dv = dg == 3 ? q : (((q + 128) & 0xFF) - 128);  // balanced digit in [-128,127]
          q = (q - dv) >> 8;
          five[dg] += dv;
          packed[dg] |= ((uint32_t)dv & 0xFFu) << (8 * b);
        }
      }
#pragma unroll
      for (int dg = 0; dg < 4; ++dg) ((uint32_t *)&piece[dg])[sl] = packed[dg];
    }
#pragma unroll
    for (int dg = 0; dg < 4; ++dg) rows[piece_offset(pc >> 4, (int)(pc & 15), R, (size_t)tok * 4 + dg) >> 4] = piece[dg];
  }
  block_sums<5>(five, shi);
  bool narrow = false;
  if (five[4] > 0) {  // uniform over the workgroup
    int bands[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int it = 0; it < TK_FUSED_HELD; ++it) {
      const size_t pc = (size_t)lane + (size_t)it * 256;
      if (pc < npieces) count_bands(held[it], shift, bands);
    }
    block_sums<8>(bands, shi);
    narrow = digits_narrow(five[4], bands);
  }
  if (lane < 4) ((int *)cst)[tok * 4 + lane] = lane == 0 ? five[0] : lane == 1 ? five[1] : lane == 2 ? five[2] : five[3];
  if (lane == 0) {
    ((int *)(cst + 256))[tok] = -shift;
    ((uint32_t *)(cst + 512))[tok] = (nonfinite || narrow) ? 1u : 0u;
  }
}

// One token whose quantization has an RMSNorm in front (the int8 contract): xs [k] and part [256] floats of LDS lie
// behind the row constants. A normalized row that holds NaN or Inf stays in xs, where the exact fallback reads it.
template <int FAST>
__device__ __forceinline__ void fused_token_a8_normed(const TkProblem &pr, uint4 *rows, uint8_t *cst, float *shf, int *shi) {
  const int lane = threadIdx.x;
  const size_t k = (size_t)pr.k, nb = (size_t)pr.nb, R = (size_t)pr.R, npieces = nb * 16;
  float *xs = (float *)(cst + 1024), *part = xs + k;
  float held[TK_FUSED_HELD][16];
#pragma unroll
  for (int it = 0; it < TK_FUSED_HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * 256;
    if (pc < npieces) load_piece_fast<FAST>(pr.raw_act, 0, piece_elem0(pc >> 4, (int)(pc & 15)), held[it]);
  }
  norm_held_pieces<TK_FUSED_HELD>(held, pr.norm_w, pr.norm_kind, pr.norm_eps, k, npieces, xs, part);
  float gamma = 0.0f;
  int nonfinite = 0;
#pragma unroll
  for (int it = 0; it < TK_FUSED_HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * 256;
    if (pc >= npieces) continue;
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      const float a = fabsf(held[it][x]);
      if (a > gamma) gamma = a;  // NaN never wins (crates/tritium-spec/src/lib.rs:351-360)
      nonfinite |= !(a <= 3.402823466e38f);
    }
  }
  block_max_any(gamma, nonfinite, shf, shi);
  const float s = gamma == 0.0f ? 0.0f : __fdiv_rn(127.0f, gamma);  // one divide
  const bool live = gamma != 0.0f && !nonfinite;
  const float sl_ = live ? s : 0.0f;
  int sum = 0;
#pragma unroll
  for (int it = 0; it < TK_FUSED_HELD; ++it) {
    const size_t pc = (size_t)lane + (size_t)it * 256;
    if (pc >= npieces) continue;
    const size_t e0 = piece_elem0(pc >> 4, (int)(pc & 15));
    uint4 piece;
    uint32_t *pw = (uint32_t *)&piece;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      if (nonfinite)  // uniform
        *(float4 *)(xs + e0 + (size_t)sl * 32) =
            make_float4(held[it][sl * 4], held[it][sl * 4 + 1], held[it][sl * 4 + 2], held[it][sl * 4 + 3]);
      uint32_t packed = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        float x = held[it][sl * 4 + b];
        if (!live) x = 0.0f;  // (a NaN or Inf times zero would not be zero)
        float r = rintf(__fmul_rn(x, sl_));  // one multiply, ties to even
        r = __builtin_fminf(__builtin_fmaxf(r, -128.0f), 127.0f);
        const int q = (int)r;
        sum += q;
        packed |= ((uint32_t)q & 0xFFu) << (8 * b);
      }
      pw[sl] = packed;
    }
    rows[piece_offset(pc >> 4, (int)(pc & 15), R, 0) >> 4] = piece;
  }
  sum = block_sum(sum, shi);
  if (lane == 0) {
    ((int *)cst)[0] = sum;
    ((float *)(cst + 256))[0] = gamma == 0.0f ? 0.0f : __fdiv_rn(gamma, 127.0f);
    ((uint32_t *)(cst + 512))[0] = nonfinite ? 1u : 0u;
    ((float *)(cst + 768))[0] = s;
  }
}

__device__ __forceinline__ void fused_stage_rows(const TkProblem &pr, uint4 *rows, uint8_t *cst) {
  __shared__ float shf[4];
  __shared__ int shi[32];
  if (pr.norm_kind) {  // (one token under the int8 contract: the host's rule)
    if (pr.raw_dtype == TK_BF16) fused_token_a8_normed<2>(pr, rows, cst, shf, shi);
    else fused_token_a8_normed<1>(pr, rows, cst, shf, shi);
    __syncthreads();
    return;
  }
  const int M = pr.M;
  const size_t k = (size_t)pr.k, nb = (size_t)pr.nb, R = (size_t)pr.R;
  const void *act = pr.raw_act;
  const bool bf16 = pr.raw_dtype == TK_BF16;
  for (int tok = 0; tok < M; ++tok) {
    if (pr.mode == TK_MODE_INT8) {
      if (bf16) fused_token_a8<2>(act, tok, k, nb, R, rows, cst, shf, shi);
      else fused_token_a8<1>(act, tok, k, nb, R, rows, cst, shf, shi);
    } else {
      if (bf16) fused_token_digits<2>(act, tok, k, nb, R, rows, cst, shf, shi);
      else fused_token_digits<1>(act, tok, k, nb, R, rows, cst, shf, shi);
    }
  }
  __syncthreads();
}

// seq_dot_raw() under the int8 contract for a row of f32 values that lies in LDS (the normalized row of the fused
// form): seq_dot_raw reads its activations with global loads, which an LDS address must never reach.
__device__ __noinline__ float seq_dot_a8_lds(const uint8_t *codes, int nb, int kdim, const float *y, int n, float s,
                                             int gamma_zero) {
  float acc = 0.0f;
  for (int k = 0; k < kdim; ++k) {
    const int code = code_at(codes, nb, n, k);
    if (code == 1) continue;
    float a = y[k];
    if (gamma_zero) {
      a = 0.0f;
    } else {
      a = rintf(__fmul_rn(a, s));
      a = a < -128.0f ? -128.0f : (a > 127.0f ? 127.0f : a);
    }
    acc = (code == 2) ? __fadd_rn(acc, a) : __fsub_rn(acc, a);
  }
  return acc;
}

// exact_rows() with the per-token constants of the fused form (in LDS, not in the problem's arrays)
__device__ __forceinline__ void exact_rows_fused(const TkProblem &pr, int n, int rowbase, unsigned flag, const uint8_t *cst) {
  if (pr.out_dtype == TK_I32) return;
  const bool a8 = pr.mode == TK_MODE_INT8;
  for (int r = 0; r < (a8 ? 4 : 1); ++r) {
    const int m = a8 ? rowbase + r : rowbase >> 2;  // the token
    if (m >= pr.M || !(flag & (1u << r))) continue;
    const float as = a8 ? ((const float *)(cst + 256))[m] : 1.0f;
    const float s = a8 ? ((const float *)(cst + 768))[m] : 0.0f;
    float f = 0.0f;
    for (int p = 0; p < pr.planes; ++p) {
      // behind an RMSNorm (one token) the row to re-quantize is the normalized one, left in LDS by the staging
      const float dot = pr.norm_kind ? seq_dot_a8_lds(pr.codes[p], pr.nb, pr.k, (const float *)(cst + 1024), n, s, as == 0.0f)
                                     : seq_dot_raw(pr.codes[p], pr.nb, pr.k, pr.raw_act, pr.raw_dtype, n, m, a8 ? 1 : 0, s, a8 && as == 0.0f);
      float t = __fmul_rn(dot, pr.scales[p][n]);
      f = p == 0 ? t : __fadd_rn(f, t);
    }
    if (a8) f = __fmul_rn(f, as);
    store_out(pr.out, pr.out_dtype, (size_t)m * pr.n + n, with_residual(pr.residual, pr.out_dtype, (size_t)m * pr.n + n, f));
  }
}

// Already-quantized int8 rows -> operand order + row sums.
__global__ __launch_bounds__(TK_WG) void tk_prep_i8_kernel(TkPrep single, const TkPrep *__restrict__ table,
                                                           int nprep, int uniform_m) {
  __shared__ int shi[4];
  int rowi;
  const TkPrep &pp = find_prep(single, table, nprep, uniform_m, rowi);
  const size_t row = rowi, k = pp.k, nb = pp.nb, R = pp.rs;
  const int8_t *q = (const int8_t *)pp.act;
  int8_t *ap = pp.ap;
  const size_t base = row * k;
  const bool vec = (k & 3) == 0 && (((size_t)q) & 3) == 0;
  int sum = 0;
  for (size_t pc = threadIdx.x; pc < nb * 16; pc += TK_WG) {
    const size_t kb = pc >> 4;
    const int q16 = (int)(pc & 15);
    const size_t e0 = piece_elem0(kb, q16);
    v4u piece;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const size_t e = e0 + (size_t)sl * 32;
      uint32_t packed = 0;
      if (vec && e + 4 <= k) {
        packed = *(const TK_GLOBAL uint32_t *)(q + base + e);
      } else {
        for (int b = 0; b < 4; ++b)
          if (e + b < k) packed |= ((uint32_t)q[base + e + b] & 0xFFu) << (8 * b);
      }
      sum += (int)(int8_t)(packed) + (int)(int8_t)(packed >> 8) + (int)(int8_t)(packed >> 16) + (int)(int8_t)(packed >> 24);
      piece[sl] = packed;
    }
    *(TK_GLOBAL v4u *)(ap + piece_offset(kb, q16, R, row)) = piece;
  }
  sum = block_sum(sum, shi);
  if (threadIdx.x == 0) pp.rowsum[row] = sum;
}

// One wave per 1-KiB chunk of a re-laid-out plane: the chunk is zero when all of its bytes are 0x55
// (rows past n were filled with that, so they do not stand in the way).
__global__ __launch_bounds__(TK_WG) void tk_zero_chunk_map_kernel(const uint8_t *__restrict__ codes, size_t chunks,
                                                                  uint32_t *__restrict__ map, unsigned *__restrict__ count) {
  const size_t chunk = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (chunk >= chunks) return;
  const uint4 v = gload16(codes + chunk * TK_CHUNK_BYTES + (size_t)(threadIdx.x & 63) * 16);
  const bool zero = v.x == 0x55555555u && v.y == 0x55555555u && v.z == 0x55555555u && v.w == 0x55555555u;
  if (__all(zero) && (threadIdx.x & 63) == 0) {
    atomicOr(map + (chunk >> 5), 1u << (chunk & 31));
    atomicAdd(count, 1u);
  }
}

__global__ void tk_copy_kernel_dev(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// ------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------

static inline unsigned grid_for(size_t total, unsigned block) { return (unsigned)((total + block - 1) / block); }

hipError_t tk_launch_relayout_tq2(hipStream_t s, const uint8_t *raw, uint8_t *codes, size_t n, size_t nb,
                                  int *invalid_row, float *block_scales) {
  size_t pieces = ((n + 15) / 16) * nb * 64;
  if (!pieces) return hipSuccess;
  hipLaunchKernelGGL(tk_relayout_tq2_kernel, dim3(grid_for(pieces, 256)), dim3(256), 0, s, raw, codes, n, nb, pieces,
                     invalid_row, block_scales);
  return hipGetLastError();
}

hipError_t tk_launch_relayout_tq1(hipStream_t s, const uint8_t *raw, uint8_t *codes, size_t n, size_t nb) {
  size_t pieces = ((n + 15) / 16) * nb * 64;
  if (!pieces) return hipSuccess;
  hipLaunchKernelGGL(tk_relayout_tq1_kernel, dim3(grid_for(pieces, 256)), dim3(256), 0, s, raw, codes, n, nb, pieces);
  return hipGetLastError();
}

hipError_t tk_launch_zero_chunk_map(hipStream_t s, const uint8_t *codes, size_t chunks, uint32_t *map, unsigned *count) {
  if (!chunks) return hipSuccess;
  hipLaunchKernelGGL(tk_zero_chunk_map_kernel, dim3(grid_for(chunks, 4)), dim3(TK_WG), 0, s, codes, chunks, map, count);
  return hipGetLastError();
}

// words of one plane's map a flow workgroup of `tiles_per_wg` tiles can touch (its chunk range may start
// and end inside a word)
size_t tk_flow_zmap_words(size_t tiles_per_wg, size_t nb) { return (tiles_per_wg * nb + 31) / 32 + 1; }

hipError_t tk_launch_decode_trits(hipStream_t s, const uint8_t *codes, size_t n, size_t k, size_t nb, int8_t *trits) {
  if (!(n * k)) return hipSuccess;
  hipLaunchKernelGGL(tk_decode_trits_kernel, dim3(grid_for(n * k, 256)), dim3(256), 0, s, codes, n, k, nb, trits);
  return hipGetLastError();
}

// Launches of up to this many tokens (quantization; the digit split, which does more per element, up to 8/3 of
// it) give a token the whole workgroup (tk_launch_prep). Measured, wave per token / workgroup per token:
// quantization K=2048 256 tokens 4.1 / 3.7 us, 512 tokens 4.2 / 4.5; K=6912 120 tokens 7.1 / 4.6, 960 tokens
// 8.8 / 9.7; digit split K=2048 512 tokens 5.9 / 5.7, 1024 tokens 8.1 / 7.0, 2048 tokens 10.7 / 11.7.
static int g_prep_team_rows = 384;
void tk_prep_set_team_rows(int rows) { g_prep_team_rows = rows < 0 ? 0 : rows; }
int tk_prep_fast(const TkPrep &pp) {
  const bool ok = pp.k % 256 == 0 && (((size_t)pp.act) & 15) == 0 && pp.ap && !pp.q_rowmajor && !pp.norm_kind && !pp.blocksum;
  if (!ok) return 0;
  return pp.act_dtype == TK_F32 ? 1 : (pp.act_dtype == TK_BF16 ? 2 : 0);
}
// ... the same for the one-pass RMSNorm + quantization kernel, which takes entries with and without a norm (at most
// 512 pieces, i.e. K <= 8192; aligned norm weights): 1 (f32) or 2 (bf16), else 0
int tk_prep_norm_fast(const TkPrep &pp) {
  const bool ok = pp.k % 256 == 0 && (((size_t)pp.act) & 15) == 0 && pp.ap && !pp.q_rowmajor && !pp.blocksum &&
                  pp.nb * 16 <= 2 * (size_t)TK_WG && (!pp.norm_kind || (pp.norm_w && (((size_t)pp.norm_w) & 15) == 0));
  if (!ok) return 0;
  return pp.act_dtype == TK_F32 ? 1 : (pp.act_dtype == TK_BF16 ? 2 : 0);
}

hipError_t tk_launch_prep(hipStream_t s, int kind, const TkPrep *single, const TkPrep *table, int nprep, int uniform_m,
                          unsigned rows, int table_wave_pieces, int table_fast, int table_norm_fast, int table_norm_pieces) {
  if (!rows) return hipSuccess;
  TkPrep dummy = {};
  const TkPrep &sg = single ? *single : dummy;
  // RMSNorm in front of the quantization, rows of whole K blocks: one pass over memory
  const int norm_fast = kind != TK_PREP_A8 ? 0 : (single ? (single->norm_kind ? tk_prep_norm_fast(*single) : 0) : table_norm_fast);
  if (norm_fast) {
    const size_t pieces = single ? single->nb * 16 : (size_t)table_norm_pieces;
    const dim3 grid(rows), block(TK_WG);
    if (pieces <= (size_t)TK_WG) {
      if (norm_fast == 2) hipLaunchKernelGGL((tk_prep_a8_norm_kernel<1, 2>), grid, block, 0, s, sg, table, nprep, uniform_m);
      else hipLaunchKernelGGL((tk_prep_a8_norm_kernel<1, 1>), grid, block, 0, s, sg, table, nprep, uniform_m);
    } else {
      if (norm_fast == 2) hipLaunchKernelGGL((tk_prep_a8_norm_kernel<2, 2>), grid, block, 0, s, sg, table, nprep, uniform_m);
      else hipLaunchKernelGGL((tk_prep_a8_norm_kernel<2, 1>), grid, block, 0, s, sg, table, nprep, uniform_m);
    }
    return hipGetLastError();
  }
  // Rows that need neither a norm nor per-block sums, whose pieces the threads working on a token can keep
  // in registers. Team = the threads of one token: a wave (four tokens per workgroup, no barrier), up to 4
  // pieces per lane (K <= 4096) or 8 in the straight-line form (whole K blocks, aligned rows of one element
  // type, operand rows only), whose registers hold little else; or, in the straight-line form, the whole
  // workgroup (up to 8 pieces per thread: K <= 32768), where few tokens make the launch one token's chain of
  // instructions (g_prep_team_rows tokens and fewer).
  const int fast = single ? tk_prep_fast(*single) : table_fast;
  size_t pieces = (size_t)(table_wave_pieces > 0 ? table_wave_pieces : 0);
  if (single) pieces = (!single->norm_kind && !single->blocksum) ? single->nb * 16 : 0;
  const bool plain = pieces && (kind == TK_PREP_A8 || kind == TK_PREP_DIGITS);
  const bool team_wg = plain && fast && pieces <= 8 * (size_t)TK_WG && (rows <= (unsigned)(kind == TK_PREP_DIGITS ? g_prep_team_rows * 8 / 3 : g_prep_team_rows) || pieces > 512);
  const bool team_wave = plain && !team_wg && rows >= 32 && pieces <= (fast ? 512u : 256u);
  if (team_wg || team_wave) {
    const size_t team = team_wg ? TK_WG : 64;
    const dim3 grid(team_wg ? rows : (rows + 3) / 4), block(TK_WG);
    const size_t per = (pieces + team - 1) / team;
    const int held = per <= 1 ? 1 : (per <= 2 ? 2 : (per <= 4 ? 4 : 8));
#define TK_WAVE_PREP(KERNEL, H, F, T) hipLaunchKernelGGL((KERNEL<H, F, T>), grid, block, 0, s, sg, table, nprep, uniform_m, rows)
#define TK_WAVE_PREP_H(KERNEL, F, T)                    \
  switch (held) {                                       \
    case 1: TK_WAVE_PREP(KERNEL, 1, F, T); break;       \
    case 2: TK_WAVE_PREP(KERNEL, 2, F, T); break;       \
    case 4: TK_WAVE_PREP(KERNEL, 4, F, T); break;       \
    default: TK_WAVE_PREP(KERNEL, 8, F, T); break;      \
  }
#define TK_WAVE_PREP_K(KERNEL)                                                         \
  if (team_wg) {                                                                       \
    if (fast == 2) { TK_WAVE_PREP_H(KERNEL, 2, 256) } else { TK_WAVE_PREP_H(KERNEL, 1, 256) } \
  } else if (fast == 2) { TK_WAVE_PREP_H(KERNEL, 2, 64) }                              \
  else if (fast == 1) { TK_WAVE_PREP_H(KERNEL, 1, 64) }                                \
  else if (held == 1) TK_WAVE_PREP(KERNEL, 1, 0, 64);                                  \
  else if (held == 2) TK_WAVE_PREP(KERNEL, 2, 0, 64);                                  \
  else TK_WAVE_PREP(KERNEL, 4, 0, 64)
    if (kind == TK_PREP_A8) {
      TK_WAVE_PREP_K(tk_prep_a8_wave_kernel);
    } else {
      TK_WAVE_PREP_K(tk_prep_digits_wave_kernel);
    }
#undef TK_WAVE_PREP_K
#undef TK_WAVE_PREP_H
#undef TK_WAVE_PREP
    return hipGetLastError();
  }
  switch (kind) {
    case TK_PREP_A8:
      if (single && single->nb * 16 <= (size_t)TK_WG)
        hipLaunchKernelGGL(tk_prep_a8_kernel<1>, dim3(rows), dim3(TK_WG), 0, s, sg, table, nprep, uniform_m);
      else if (single && single->nb * 16 <= 2 * (size_t)TK_WG)
        hipLaunchKernelGGL(tk_prep_a8_kernel<2>, dim3(rows), dim3(TK_WG), 0, s, sg, table, nprep, uniform_m);
      else
        hipLaunchKernelGGL(tk_prep_a8_kernel<TK_PREP_HELD>, dim3(rows), dim3(TK_WG), 0, s, sg, table, nprep, uniform_m);
      break;
    case TK_PREP_DIGITS: hipLaunchKernelGGL(tk_prep_digits_kernel, dim3(rows), dim3(TK_WG), 0, s, sg, table, nprep, uniform_m); break;
    case TK_PREP_I8: hipLaunchKernelGGL(tk_prep_i8_kernel, dim3(rows), dim3(TK_WG), 0, s, sg, table, nprep, uniform_m); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

template <int P>
static hipError_t launch_skinny_p(hipStream_t s, const TkProblem *single, const TkProblem *table, int nprobs,
                                  const TkLaunchCfg &cfg) {
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  dim3 grid(cfg.grid), block(TK_WG);
  if (cfg.fused) {  // the operand rows are built inside the kernel: one row tile
    if (cfg.rt != 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL((tk_skinny_kernel<P, 1, true>), grid, block, cfg.lds_bytes, s, sg, table, nprobs);
    return hipGetLastError();
  }
  switch (cfg.rt) {
    case 1: hipLaunchKernelGGL((tk_skinny_kernel<P, 1>), grid, block, cfg.lds_bytes, s, sg, table, nprobs); break;
    case 2: hipLaunchKernelGGL((tk_skinny_kernel<P, 2>), grid, block, cfg.lds_bytes, s, sg, table, nprobs); break;
    case 4: hipLaunchKernelGGL((tk_skinny_kernel<P, 4>), grid, block, cfg.lds_bytes, s, sg, table, nprobs); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t tk_launch_skinny(hipStream_t s, const TkProblem *single, const TkProblem *table, int nprobs,
                            const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  switch (cfg.planes) {
    case 1: return launch_skinny_p<1>(s, single, table, nprobs, cfg);
    case 2: return launch_skinny_p<2>(s, single, table, nprobs, cfg);
    case 3: return launch_skinny_p<3>(s, single, table, nprobs, cfg);
    case 4: return launch_skinny_p<4>(s, single, table, nprobs, cfg);
    default: return hipErrorInvalidValue;
  }
}

template <int P, int RT>
static hipError_t launch_stream_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                   const TkLaunchCfg &cfg) {
  constexpr int TW = (P * RT <= 4) ? 4 : ((P * RT <= 8) ? 2 : 1);
  hipLaunchKernelGGL((tk_stream_kernel<P, RT, TW>), dim3(cfg.grid), dim3(TK_WG), cfg.lds_bytes, s, sg, table, wg_prob);
  return hipGetLastError();
}

template <int P>
static hipError_t launch_stream_p(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                  const TkLaunchCfg &cfg) {
  switch (cfg.rt) {
    case 1: return launch_stream_pr<P, 1>(s, sg, table, wg_prob, cfg);
    case 2: return launch_stream_pr<P, 2>(s, sg, table, wg_prob, cfg);
    case 4: return launch_stream_pr<P, 4>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

int tk_stream_tiles_per_wg(int planes, int rt) {
  const int pr = planes * rt;
  return 4 * (pr <= 4 ? 4 : (pr <= 8 ? 2 : 1));
}

hipError_t tk_launch_stream(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                            const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  switch (cfg.planes) {
    case 1: return launch_stream_p<1>(s, sg, table, wg_prob, cfg);
    case 2: return launch_stream_p<2>(s, sg, table, wg_prob, cfg);
    case 3: return launch_stream_p<3>(s, sg, table, wg_prob, cfg);
    case 4: return launch_stream_p<4>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

template <int P, int RT>
static hipError_t launch_flow_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                 const TkLaunchCfg &cfg) {
  constexpr int TW = ((RT >= 4 && P <= 2) || (RT == 2 && P == 1)) ? 2 : 1;
  const int threads = cfg.waves * 64;
  if constexpr (RT == 1) {
    if (cfg.fused) {  // the operand rows are built inside the kernel: 256 threads; from a table for one or two planes
      if (threads != 256) return hipErrorInvalidValue;
      if constexpr (P <= 2) {
        if (cfg.tw == 2) {
          switch (cfg.ring) {
            case 2: return table ? flow_launch_one(tk_flow_kernel<P, 1, 2, 2, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 2, 2, false, true>, s, sg, table, wg_prob, cfg, threads);
            case 3: return table ? flow_launch_one(tk_flow_kernel<P, 1, 2, 3, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 2, 3, false, true>, s, sg, table, wg_prob, cfg, threads);
            case 4: return table ? flow_launch_one(tk_flow_kernel<P, 1, 2, 4, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 2, 4, false, true>, s, sg, table, wg_prob, cfg, threads);
            case 5: return table ? flow_launch_one(tk_flow_kernel<P, 1, 2, 5, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 2, 5, false, true>, s, sg, table, wg_prob, cfg, threads);
            default: return hipErrorInvalidValue;
          }
        }
        switch (cfg.ring) {
          case 2: return table ? flow_launch_one(tk_flow_kernel<P, 1, 1, 2, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 1, 2, false, true>, s, sg, table, wg_prob, cfg, threads);
          case 3: return table ? flow_launch_one(tk_flow_kernel<P, 1, 1, 3, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 1, 3, false, true>, s, sg, table, wg_prob, cfg, threads);
          case 4: return table ? flow_launch_one(tk_flow_kernel<P, 1, 1, 4, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 1, 4, false, true>, s, sg, table, wg_prob, cfg, threads);
          case 5: return table ? flow_launch_one(tk_flow_kernel<P, 1, 1, 5, true, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, 1, 1, 5, false, true>, s, sg, table, wg_prob, cfg, threads);
          default: return hipErrorInvalidValue;
        }
      }
      if (table) return hipErrorInvalidValue;
      switch (cfg.ring) {
        case 2: return flow_launch_one(tk_flow_kernel<P, 1, 1, 2, false, true>, s, sg, table, wg_prob, cfg, threads);
        case 3: return flow_launch_one(tk_flow_kernel<P, 1, 1, 3, false, true>, s, sg, table, wg_prob, cfg, threads);
        case 4: return flow_launch_one(tk_flow_kernel<P, 1, 1, 4, false, true>, s, sg, table, wg_prob, cfg, threads);
        case 5: return flow_launch_one(tk_flow_kernel<P, 1, 1, 5, false, true>, s, sg, table, wg_prob, cfg, threads);
        default: return hipErrorInvalidValue;
      }
    }
  }
  if constexpr (P <= 2 && RT == 1) {  // one row tile: one or two runs per wave, the host's choice by row count
    if (cfg.tw == 2) {
      switch (cfg.ring) {
        case 2: return table ? flow_launch_one(tk_flow_kernel<P, RT, 2, 2, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, RT, 2, 2, false>, s, sg, table, wg_prob, cfg, threads);
        case 3: return table ? flow_launch_one(tk_flow_kernel<P, RT, 2, 3, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, RT, 2, 3, false>, s, sg, table, wg_prob, cfg, threads);
        case 4: return table ? flow_launch_one(tk_flow_kernel<P, RT, 2, 4, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, RT, 2, 4, false>, s, sg, table, wg_prob, cfg, threads);
        case 5: return table ? flow_launch_one(tk_flow_kernel<P, RT, 2, 5, true>, s, sg, table, wg_prob, cfg, threads) : flow_launch_one(tk_flow_kernel<P, RT, 2, 5, false>, s, sg, table, wg_prob, cfg, threads);
        default: return hipErrorInvalidValue;
      }
    }
  }
  switch (cfg.ring) {
    case 2:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 2, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 2, false>, s, sg, table, wg_prob, cfg, threads);
    case 3:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 3, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 3, false>, s, sg, table, wg_prob, cfg, threads);
    case 4:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 4, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 4, false>, s, sg, table, wg_prob, cfg, threads);
    case 5:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 5, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 5, false>, s, sg, table, wg_prob, cfg, threads);
    default: return hipErrorInvalidValue;
  }
}

template <int P, int RT2>
static hipError_t launch_flow32_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                   const TkLaunchCfg &cfg) {
  const int threads = cfg.waves * 64;
  switch (cfg.ring) {
    case 2:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 2, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 2, false>, s, sg, table, wg_prob, cfg, threads);
    case 3:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 3, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 3, false>, s, sg, table, wg_prob, cfg, threads);
    case 4:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 4, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 4, false>, s, sg, table, wg_prob, cfg, threads);
    default: return hipErrorInvalidValue;
  }
}

template <int P>
static hipError_t launch_flow_p(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                const TkLaunchCfg &cfg) {
  if (cfg.wide_mfma) {
    if constexpr (P <= 2) {
      switch (cfg.rt) {
        case 2: return launch_flow32_pr<P, 1>(s, sg, table, wg_prob, cfg);
        case 4: return launch_flow32_pr<P, 2>(s, sg, table, wg_prob, cfg);
        default: return hipErrorInvalidValue;
      }
    } else {
      return hipErrorInvalidValue;
    }
  }
  switch (cfg.rt) {
    case 1: return launch_flow_pr<P, 1>(s, sg, table, wg_prob, cfg);
    case 2: return launch_flow_pr<P, 2>(s, sg, table, wg_prob, cfg);
    case 4: return launch_flow_pr<P, 4>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

// lock-step runs per wave of the flow kernel for a (planes, rt, rows) triple: two where registers allow and a
// single run would keep too few bytes in flight (four row tiles of one or two planes; two row
// tiles of one plane: K=2048 N=8192, 32 int8 rows, one plane went from 263 to 228 us)
int tk_flow_runs_per_wave(int planes, int rt, int rows) {
  // One row tile: a second run doubles the loads a wave keeps in flight and costs registers, i.e. waves
  // per SIMD. Measured over 128 layer copies per launch: one plane (K=2560 N=6912) 4 / 4 / 16 rows
  // +5% / +10% / +7% with two runs, a single row -1.5%; two planes (K=2048 N=8192) 4..8 rows -3%,
  // 16 rows +2.4%.
  if (rt == 1) return (planes == 1 && rows >= 2) || (planes == 2 && rows >= 9) ? 2 : 1;
  return ((rt >= 4 && planes <= 2) || (rt == 2 && planes == 1)) ? 2 : 1;
}
// ... of the 32x32x32 form: always a pair of adjacent tiles
int tk_flow32_runs_per_wave(void) { return 2; }

// Ring size of the flow kernel (2..5 positions) for launches whose K block counts are nbs[0..count).
// A deeper ring keeps more loads in flight per wave and costs registers, i.e. waves per SIMD.
// Measured on K=2048 N=8192 x 2 planes: one and two row tiles like 4 positions (with runs of a
// single tile, 4 beat 5 by 5% at 4-8 operand rows), four row tiles (250 registers, eight waves per CU
// whatever the ring) 2. A ring that does not divide a K block count pads that problem's tiles with
// idle positions; a candidate is taken in the order of preference unless it pads more than a tenth
// (one row tile: K=2560 runs 2% faster on 5 positions than on 4 padded to 12) or a quarter (more
// row tiles) of the positions, weighted by each problem's chunk count; if all do, the one that
// pads least.
int tk_flow_ring(const int *nbs, const double *weights, int count, int rt, int rows, int tw) {
  // one row tile: 4 positions, and 2 where 4 would pad the K block count by more than a tenth. Re-measured with the
  // weight stream on non-temporal loads, 128 layer copies per launch: ten K blocks (K = 2560, one plane) on 2 positions
  // against 4 padded to 12 -- 6912 outputs, one f32 token 5.90 -> 6.27 TB/s, 4 / 16 int8 tokens 5.31 -> 5.61 / 4.96 ->
  // 5.16; 2560 outputs 5.55 -> 6.12, 5.29 -> 5.68, 4.61 -> 4.90 -- and 5 positions, the choice before, lose 5-14% to 2;
  // eight K blocks are within 1.5% either way (two planes, K = 2048: 2 positions +2.6% for one float token, -1% for two).
  const int pref1a[4] = {4, 2, 3, 5}, pref1b[4] = {5, 4, 3, 2}, pref2[4] = {4, 2, 3, 5}, pref4[4] = {2, 3, 4, 5};
  const int *pref1 = rows <= 8 ? pref1a : pref1b;  // (one plane with two runs per wave: the first list at every row count; see the caller)
  // two row tiles likewise: 32 int8 rows, K = 2560, one plane, 2 positions against 4 padded to 12: 6912 outputs 4.16 ->
  // 4.35 TB/s, 2560 outputs 3.91 -> 4.35, 640 outputs 2.31 -> 3.17
  const double limit = rt <= 2 ? 0.10 : 0.25;
  const int *cand = rt == 1 ? (tw >= 2 ? pref2 : pref1) : (rt == 2 ? pref2 : pref4);
  int best = cand[0];
  double best_waste = -1.0;
  for (int c = 0; c < 4; ++c) {
    double waste = 0.0, total = 0.0;
    for (int x = 0; x < count; ++x) {
      const int nb = nbs[x], pad = (nb + cand[c] - 1) / cand[c] * cand[c];
      const double w = weights ? weights[x] : 1.0;
      waste += w * (double)(pad - nb) / (double)(pad > 0 ? pad : 1);
      total += w;
    }
    waste = total > 0.0 ? waste / total : 0.0;
    if (waste <= limit) return cand[c];
    if (best_waste < 0.0 || waste < best_waste) {
      best_waste = waste;
      best = cand[c];
    }
  }
  return best;
}

hipError_t tk_launch_flow(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                          const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  if (cfg.wide_mfma && cfg.zmap32) return tk_launch_flow32_zmap(s, single, table, wg_prob, cfg);
  if (cfg.swap && !cfg.fused) return tk_launch_flow_swapped(s, single, table, wg_prob, cfg);
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  switch (cfg.planes) {
    case 1: return launch_flow_p<1>(s, sg, table, wg_prob, cfg);
    case 2: return launch_flow_p<2>(s, sg, table, wg_prob, cfg);
    case 3: return launch_flow_p<3>(s, sg, table, wg_prob, cfg);
    case 4: return launch_flow_p<4>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

// output tiles per workgroup of the GEMM for a plane count
int tk_gemm_lds_bytes(void) { return (TK_GEMM32_STAGES > 3 ? TK_GEMM32_STAGES : 3) * 16 * 64 * 16 + 1024; }  // the A blocks + the row constants
int tk_gemm_tiles_per_wg(int planes) { return TK_GEMM_WAVES * (planes == 1 ? 4 : (planes <= 3 ? 2 : 1)); }

template <typename K>
static hipError_t gemm_launch_one(K kernel, hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                  const TkLaunchCfg &cfg, unsigned wgs) {
  if (cfg.lds_bytes > 64 * 1024) {
    // (not the full 160 KiB: the kernel also has a few static bytes)
    hipError_t e = tk_raise_lds_limit((const void *)kernel, 128 * 1024);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, dim3(wgs), dim3(TK_GEMM_THREADS), cfg.lds_bytes, s, sg, table, wg_prob);
  return hipGetLastError();
}

// single != null: one problem, grid from its XCD split. table != null: a grouped launch of cfg.grid
// workgroups (every member's share is a multiple of 8).
hipError_t tk_launch_gemm(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                          const TkLaunchCfg &cfg) {
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  const bool ksplit = !table && sg.ksplit > 1;
  const unsigned wgs = table ? cfg.grid : 8u * (unsigned)sg.sub_m * (unsigned)sg.sub_n * (ksplit ? (unsigned)sg.ksplit : 1u);
  if (!wgs) return hipSuccess;
  if (ksplit) {
    if (cfg.planes == 1 && cfg.gemm_nt == 2) {
      if (!cfg.gemm_two_by_two) return gemm_launch_one(tk_gemm32_kernel<1, 2, false, true>, s, sg, table, wg_prob, cfg, wgs);
      return gemm_launch_one(tk_gemm32_kernel<1, 4, false, true, 2>, s, sg, table, wg_prob, cfg, wgs);
    }
    switch (cfg.planes) {
      case 1: return gemm_launch_one(tk_gemm32_kernel<1, 4, false, true>, s, sg, table, wg_prob, cfg, wgs);
      case 2: return gemm_launch_one(tk_gemm32_kernel<2, 2, false, true>, s, sg, table, wg_prob, cfg, wgs);
      case 3: return gemm_launch_one(tk_gemm32_kernel<3, 2, false, true>, s, sg, table, wg_prob, cfg, wgs);
      default: return hipErrorInvalidValue;  // four planes take the 16x16x64 kernel, which has no K split
    }
  }
  dim3 grid(wgs), block(TK_GEMM_THREADS);
#define TK_GEMM_CASE(PP, NTT)                                                                                 \
  if (table) hipLaunchKernelGGL((tk_gemm_kernel<PP, NTT, true>), grid, block, cfg.lds_bytes, s, sg, table, wg_prob); \
  else hipLaunchKernelGGL((tk_gemm_kernel<PP, NTT, false>), grid, block, cfg.lds_bytes, s, sg, table, wg_prob);      \
  break;
#define TK_GEMM32_CASE(PP, NTT)                                                                              \
  if (table) return gemm_launch_one(tk_gemm32_kernel<PP, NTT, true>, s, sg, table, wg_prob, cfg, wgs);        \
  return gemm_launch_one(tk_gemm32_kernel<PP, NTT, false>, s, sg, table, wg_prob, cfg, wgs);
  if (cfg.planes == 1 && cfg.gemm_nt == 2) {  // 64 x 128 outputs per workgroup: four waves side by side, or two by two
    if (!cfg.gemm_two_by_two) {
      if (table) return gemm_launch_one(tk_gemm32_kernel<1, 2, true>, s, sg, table, wg_prob, cfg, wgs);
      return gemm_launch_one(tk_gemm32_kernel<1, 2, false>, s, sg, table, wg_prob, cfg, wgs);
    }
    if (table) return gemm_launch_one(tk_gemm32_kernel<1, 4, true, false, 2>, s, sg, table, wg_prob, cfg, wgs);
    return gemm_launch_one(tk_gemm32_kernel<1, 4, false, false, 2>, s, sg, table, wg_prob, cfg, wgs);
  }
  switch (cfg.planes) {
    case 1: TK_GEMM32_CASE(1, 4)
    case 2: TK_GEMM32_CASE(2, 2)
    case 3: TK_GEMM32_CASE(3, 2)
    case 4: TK_GEMM_CASE(4, 1)
    default: return hipErrorInvalidValue;
  }
#undef TK_GEMM_CASE
#undef TK_GEMM32_CASE
  return hipGetLastError();
}

template <int P>
static hipError_t launch_salt_p(hipStream_t s, const TkProblem &sg, const TkLaunchCfg &cfg) {
  TkLaunchCfg c = cfg;
  auto go = [&](auto kernel) {
    if (c.lds_bytes > 64 * 1024) {
      hipError_t e = tk_raise_lds_limit((const void *)kernel, 160 * 1024);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, dim3(c.grid), dim3(c.waves * 64), c.lds_bytes, s, sg);
    return hipGetLastError();
  };
  switch (cfg.rt) {
    // three ring positions for every row-tile count: the depths the plain flow kernel likes
    // (5 / 4 / 2) measured 2-7% slower here
    case 1: return go(tk_salt_flow_kernel<P, 1, 3>);
    case 2: return go(tk_salt_flow_kernel<P, 2, 3>);
    case 4: return go(tk_salt_flow_kernel<P, 4, 3>);
    default: return hipErrorInvalidValue;
  }
}

hipError_t tk_launch_salt_flow(hipStream_t s, const TkProblem *single, const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  switch (cfg.planes) {
    case 1: return launch_salt_p<1>(s, *single, cfg);
    case 2: return launch_salt_p<2>(s, *single, cfg);
    case 3: return launch_salt_p<3>(s, *single, cfg);
    case 4: return launch_salt_p<4>(s, *single, cfg);
    default: return hipErrorInvalidValue;
  }
}

hipError_t tk_launch_salt_seq(hipStream_t s, const TkProblem *single) {
  size_t total = (size_t)single->M * single->n;
  if (!total) return hipSuccess;
  hipLaunchKernelGGL(tk_salt_seq_kernel, dim3(grid_for(total, TK_WG)), dim3(TK_WG), 0, s, *single);
  return hipGetLastError();
}

hipError_t tk_launch_seq(hipStream_t s, const TkProblem *single) {
  size_t total = (size_t)single->M * single->n;
  if (!total) return hipSuccess;
  hipLaunchKernelGGL(tk_seq_kernel, dim3(grid_for(total, TK_WG)), dim3(TK_WG), 0, s, *single);
  return hipGetLastError();
}

hipError_t tk_launch_copy(hipStream_t s, void *dst, const void *src, size_t bytes) {
  size_t n16 = bytes / 16;
  if (!n16) return hipSuccess;
  unsigned grid = (unsigned)((n16 + 255) / 256);
  if (grid > 256 * 32) grid = 256 * 32;
  hipLaunchKernelGGL(tk_copy_kernel_dev, dim3(grid), dim3(256), 0, s, (uint4 *)dst, (const uint4 *)src, n16);
  return hipGetLastError();
}
