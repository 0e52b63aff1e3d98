// The bandwidth kernels of the decode path (16x16x64 and 32x32x32 forms) as templates, shared by the translation
// unit that instantiates the plain forms (tk_kernels.hip) and the one that instantiates the forms of the 32x32x32
// kernel that consult the zero-chunk maps (tk_zskip.hip).
#pragma once

#include "tk_internal.h"

#include "tk_device.h"

__device__ __forceinline__ void fused_stage_rows(const TkProblem &pr, uint4 *rows, uint8_t *cst);
__device__ __forceinline__ RowConst row_const_from_lds(const uint8_t *cst, int mode, int R, int M, int rowbase);
__device__ __forceinline__ void exact_rows_fused(const TkProblem &pr, int n, int rowbase, unsigned flag, const uint8_t *cst);

// ------------------------------------------------------------------------------------------
// decode GEMV, flow form: the bandwidth kernel. Requirements: all K blocks of the operand rows fit
// in LDS. A wave owns TW runs of S output tiles; in the device layout the chunks of consecutive
// tiles are consecutive in memory, so a run is a byte stream with a fixed skip at tile starts,
// walked with a ring of 128-bit loads that never drains at tile boundaries. Per-row constants are
// loaded once per wave, per-tile scales at the start of the tile, so the epilogue of a tile waits
// on nothing that was issued behind the stream's prefetches.
// ------------------------------------------------------------------------------------------


// Waves per SIMD the register allocation must leave room for: two follow from the workgroup size (up to
// eight waves); the form with two planes and two runs per wave on a ring of four sits at the edge of
// three (168 registers) -- left alone it takes 169, which costs a third of the waves in flight and 8% of
// the rate at 9..16 operand rows.
// Workgroups of sixteen waves (a CU whose LDS holds the rows of one workgroup only then still runs four waves per SIMD)
// exist for the forms that stay within 128 registers by themselves: two row tiles of one or two planes on a ring of
// two, with weights first (107 / 100 registers) or, activations first, from a problem table (126 / 124; the form for a
// single problem takes 149).
#define TK_FLOW_MAX_THREADS(P, RT, DR, TABLE, SWAP) \
  (((RT) == 2 && ((P) <= 2 || ((P) == 3 && (SWAP))) && (DR) == 2 && ((SWAP) || (TABLE))) ? 1024 : 512)
#define TK_FLOW_MIN_WAVES(P, RT, TW, DR, SWAP) ((!(SWAP) && (P) == 2 && (RT) == 1 && (TW) == 2 && (DR) == 4) ? 3 : 2)
// FUSED (one row tile, 256 threads; a single problem or, from a table, one token per member): the kernel builds the operand rows of its one to four
// tokens itself from pr.raw_act -- see fused_stage_rows -- and the call is one launch instead of two.
// SWAP (int8 contract only; instantiated in tk_flow_a8.hip): the two operands of the matrix instruction change places --
// weights first, activations second -- so that an accumulator register holds four consecutive OUTPUT CHANNELS of one
// token (lane (g, i): token rt*16 + i, channels 16*tile + 4g .. 4g+3) instead of four tokens of one channel. The integers
// are the same; what changes is the epilogue: a lane writes its four values with ONE 8- or 16-byte store instead of
// four 2- or 4-byte stores to four output rows, and a decode launch of 8..64 tokens is held back by the number of
// store instructions it issues, not by their bytes.
template <int P, int RT, int TW, int DR, bool TABLE, bool FUSED = false, bool SWAP = false>
__global__ __launch_bounds__(TK_FLOW_MAX_THREADS(P, RT, DR, TABLE, SWAP)) __attribute__((amdgpu_waves_per_eu(TK_FLOW_MIN_WAVES(P, RT, TW, DR, SWAP)))) void tk_flow_kernel(const TkProblem single, const TkProblem *__restrict__ table,
                                                      const int *__restrict__ wg_prob) {
  static_assert(!FUSED || RT == 1, "the fused form: one row tile");
  static_assert(!(FUSED && SWAP), "the fused form keeps the first operand order");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const TkProblem &pr = TABLE ? table[wg_prob[blockIdx.x]] : *single_problem();
  const int NW = (int)(blockDim.x >> 6);  // 4 or 8 waves
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int nb = pr.nb, R = pr.R, S = pr.run_tiles, n_tiles = pr.n_tiles;
  // local copies: a field read through the table pointer would be fetched again after every store
  const TkHot hot = make_hot(pr);
  const uint8_t *codes[P];
  const float *scales[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    codes[p] = pr.codes[p];
    scales[p] = pr.scales[p];
  }
  // The weight stream of a run is walked in positions q = s*nbpad + kb, nbpad = nb rounded up to a
  // multiple of the ring size DR (positions kb >= nb are padding: nothing is computed there). Slot =
  // kb % DR. At EVERY position, padding included, the chunks D = DR-1 positions ahead are requested
  // into the slot consumed one position ago: no register is copied, no chunk is overwritten before
  // its use, and because each position issues the same number of loads the wait in front of a
  // chunk's first use leaves exactly the D younger positions in flight. The chunks of a run are
  // consecutive in memory, so a request is one running byte offset per run, advanced by 1 KiB when
  // the requested position is a real one; a padding position asks again for the chunk the next real
  // position will get, and requests past the end of the run ask again for its last chunk (a cache
  // hit: no traffic from memory). The host picks DR so that padding is rare.
  constexpr int D = DR - 1;
  const int nbpad = (nb + DR - 1) / DR * DR;
  const int first = ((blockIdx.x - pr.group_begin) * NW + wave) * TW * S;  // first tile of this wave
  const unsigned plane_last = (unsigned)n_tiles * (unsigned)nb - 1u;  // last chunk of the plane
  // The TW runs of a wave interleave tile by tile (run tw takes tiles first+tw, first+tw+TW, ...), so
  // that what the wave finishes together is TW*16 adjacent output columns (its stores then fill
  // whole cache lines between them); at the first position of a tile a run therefore skips the
  // (TW-1) tiles of its siblings.
  const unsigned skip = (unsigned)(TW - 1) * (unsigned)nb * 1024u;
  unsigned roff[TW];      // byte offset inside a plane of this lane's piece of the next chunk to request
  unsigned last_off[TW];  // ... of the last chunk of the run: requests past it ask for that chunk again
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    roff[tw] = (unsigned)(first + tw) * (unsigned)nb * 1024u + (unsigned)lane * 16u - skip;
    const unsigned run_last = (unsigned)(first + (S - 1) * TW + tw) * (unsigned)nb + (unsigned)nb - 1u;
    last_off[tw] = min(run_last, plane_last) * 1024u + (unsigned)lane * 16u;
  }

  // Zero-chunk skip: the map words of the chunks this workgroup can ask for sit in LDS behind the
  // operand rows (staged below); a request for a chunk whose bit is set goes to the all-zero chunk
  // that follows the plane's last chunk -- the same bytes from the cache instead of from memory, so
  // neither the arithmetic nor the number of loads per position changes. The ring's first requests are
  // issued before that staging and read their map words from memory (with runs of one tile they are
  // three of a tile's eight chunks: left unmapped, a plane with 75% zero chunks fetched 23% less instead
  // of 37%).
  const bool zskip = !FUSED && pr.zskip != 0;  // (the fused form keeps its row constants where the maps would go)
  const uint32_t *lds_z = (const uint32_t *)(smem + (size_t)nb * 256 * R);
  const unsigned zero_off = (unsigned)n_tiles * (unsigned)nb * 1024u + (unsigned)lane * 16u;
  const unsigned wg_first = (unsigned)(blockIdx.x - pr.group_begin) * (unsigned)(NW * TW * S);
  const unsigned zc0 = min(wg_first, (unsigned)n_tiles - 1u) * (unsigned)nb;
  const unsigned zc1 = min(wg_first + (unsigned)(NW * TW * S), (unsigned)n_tiles) * (unsigned)nb;  // exclusive
  const unsigned zw0 = zc0 >> 5, zwords = zskip ? ((max(zc1, zc0 + 1u) - 1u) >> 5) - zw0 + 1u : 0u;
  uint4 ring[DR][TW][P];
  auto request = [&](int slot, bool real, bool tile_start, bool use_map) {
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      roff[tw] += tile_start ? skip : 0u;
      const unsigned off = min(roff[tw], last_off[tw]);
#pragma unroll
      for (int p = 0; p < P; ++p) {
        unsigned o = off;
        if (zskip) {
          const unsigned chunk = (unsigned)__builtin_amdgcn_readfirstlane((int)(off >> 10));
          uint32_t word;
          if (use_map) {
            const unsigned wi = (chunk >> 5) - zw0;
            word = wi < zwords ? lds_z[(unsigned)p * zwords + wi] : 0u;
          } else {  // the first requests of a workgroup, before its map words are in LDS: straight from memory
            const uint32_t *zm = pr.zmap[p];
            word = zm ? gload(zm + (chunk >> 5)) : 0u;
          }
          if ((word >> (chunk & 31u)) & 1u) o = zero_off + ((chunk & (unsigned)(TK_ZERO_CHUNKS - 1)) << 10);
        }
        ring[slot][tw][p] = gload16_stream(codes[p] + (size_t)o);
      }
      roff[tw] += real ? 1024u : 0u;
    }
  };
#pragma unroll
  for (int d = 0; d < D; ++d) request(d, d < nb, d == 0, false);  // (the map is not staged yet: read from memory)

  // stage every operand row of the problem in LDS
  uint8_t *const cst = smem + (size_t)nb * 256 * R;  // fused form: the row constants behind the rows
  if constexpr (FUSED) {
    fused_stage_rows(pr, (uint4 *)smem, cst);
  } else {
    const uint4 *ap4 = (const uint4 *)pr.ap;
    uint4 *lds4w = (uint4 *)smem;
    const int cnt = nb * 16 * R;
    for (int idx = threadIdx.x; idx < cnt; idx += (int)blockDim.x) lds4w[idx] = gload16(ap4 + idx);
    if (zskip) {
      uint32_t *lz = (uint32_t *)(smem + (size_t)nb * 256 * R);
      for (unsigned idx = threadIdx.x; idx < (unsigned)P * zwords; idx += blockDim.x) {
        const unsigned p = idx / zwords, w = idx - p * zwords;
        lz[idx] = pr.zmap[p] ? gload(pr.zmap[p] + zw0 + w) : 0u;
      }
    }
  }
  RowConst rc[RT];
  unsigned any_flag = 0;
  // SWAP: the constants of this lane's one token per row tile (row rt*16 + i)
  int tok_rs[RT];
  float tok_as[RT];
  unsigned tok_flag[RT];
  if constexpr (SWAP) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int m = rt * 16 + i;
      tok_rs[rt] = m < R ? gload(hot.rowsum + m) : 0;
      tok_as[rt] = m < R && hot.act_scale ? gload(hot.act_scale + m) : 1.0f;
      tok_flag[rt] = m < R && hot.flags ? gload(hot.flags + m) : 0u;
      any_flag |= tok_flag[rt];
    }
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if constexpr (FUSED) rc[rt] = row_const_from_lds(cst, hot.mode, R, hot.M, rt * 16 + 4 * g);  // (staged behind a barrier)
      else rc[rt] = load_row_const(hot, rt * 16 + 4 * g);
      any_flag |= rc[rt].flag;
    }
  }
  if constexpr (!FUSED) __syncthreads();
  const uint4 *lds4 = (const uint4 *)smem;
  // operand rows past R re-read the last row: their results are never stored
  int arow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) arow[rt] = min(rt * 16 + i, R - 1);

  for (int s = 0; s < S; ++s) {
    // per-tile scales, issued now, consumed in the epilogue
    float sc[TW][P];
    // SWAP: the scales of this lane's four channels (requested behind the K loop instead, they save the two-plane forms
    // nine registers and cost every form 2-7%: the epilogue then waits for them)
    float sc4[SWAP ? TW : 1][SWAP ? P : 1][4];
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      if constexpr (SWAP) {
        const int n0 = (first + s * TW + tw) * 16 + 4 * g;
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
          for (int r = 0; r < 4; ++r) sc4[tw][p][r] = gload(scales[p] + min(n0 + r, hot.n - 1));
      } else {
        const int n = min((first + s * TW + tw) * 16 + i, hot.n - 1);
#pragma unroll
        for (int p = 0; p < P; ++p) sc[tw][p] = gload(scales[p] + n);
      }
    }
    v4i acc[TW][RT][P];
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int p = 0; p < P; ++p) acc[tw][rt][p] = v4i{0, 0, 0, 0};

    // a do-while: K has at least one block, and without a way round the loop the waits of the epilogue
    // (for the scales requested above) can leave the ring's youngest requests in flight
    int kbg = 0;
    do {
#pragma unroll
      for (int d = 0; d < DR; ++d) {
        const int kb = kbg + d;
        {  // request the position D ahead (slot (d + D) % DR, consumed at the previous position)
          int kb2 = kb + D;
          if (kb2 >= nbpad) kb2 -= nbpad;
          request((d + D) % DR, kb2 < nb, kb2 == 0, true);
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
            for (int tw = 0; tw < TW; ++tw)
#pragma unroll
              for (int p = 0; p < P; ++p) {
                const uint4 w = ring[d][tw][p];
                const uint32_t wj = j == 0 ? w.x : (j == 1 ? w.y : (j == 2 ? w.z : w.w));
                const v4i b = expand_codes(wj);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                  acc[tw][rt][p] = SWAP ? __builtin_amdgcn_mfma_i32_16x16x64_i8(b, a[rt], acc[tw][rt][p], 0, 0, 0)
                                        : __builtin_amdgcn_mfma_i32_16x16x64_i8(a[rt], b, acc[tw][rt][p], 0, 0, 0);
              }
          }
        }
      }
      kbg += DR;
    } while (kbg < nbpad);

    if constexpr (SWAP) {
#pragma unroll
      for (int tw = 0; tw < TW; ++tw) {
        const int t = first + s * TW + tw;
        const int n0 = t * 16 + 4 * g;
        if (t < n_tiles && n0 < hot.n) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            flow_epilogue_swapped<P>(hot, pr, rt * 16 + i, n0, acc[tw][rt], sc4[tw], tok_rs[rt], tok_as[rt], tok_flag[rt]);
        }
      }
      continue;
    }
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      const int t = first + s * TW + tw;
      const int n = t * 16 + i;
      if (t < n_tiles && n < hot.n) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) flow_epilogue<P>(hot, n, rt * 16 + 4 * g, acc[tw][rt], sc[tw], rc[rt]);
      }
    }
    if (any_flag) {
      for (int tw = 0; tw < TW; ++tw) {
        const int t = first + s * TW + tw;
        const int n = t * 16 + i;
        if (t >= pr.n_tiles || n >= pr.n) continue;
        for (int rt = 0; rt < RT; ++rt) {
          const int rowbase = rt * 16 + 4 * g;
          if constexpr (FUSED) {
            if (rc[rt].flag) exact_rows_fused(pr, n, rowbase, rc[rt].flag, cst);
          } else {
            const unsigned fl = row_flags(pr, rowbase);
            if (fl) exact_rows(pr, n, rowbase, fl);
          }
        }
      }
    }
  }
}

// Row constants of the 4 operand rows starting at rowbase from a copy in LDS
// (int rowsum[64] | float scale or int exponent [64] | uint flag[64]).
__device__ __forceinline__ RowConst row_const_from_lds(const uint8_t *cst, int mode, int R, int M, int rowbase) {
  const int *cst_rs = (const int *)cst;
  const float *cst_as = (const float *)(cst + 256);
  const int *cst_exp = (const int *)(cst + 256);
  const uint32_t *cst_flag = (const uint32_t *)(cst + 512);
  RowConst rc;
  rc.exp = 0;
  rc.flag = 0;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = rowbase + r;
    rc.rs[r] = m < R ? cst_rs[m] : 0;
    rc.as[r] = 1.0f;
  }
  if (mode == TK_MODE_INT8) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = rowbase + r;
      if (m < R) {
        rc.as[r] = cst_as[m];
        if (cst_flag[m]) rc.flag |= 1u << r;
      }
    }
  } else {
    const int tok = rowbase >> 2;
    if (tok < M) {
      rc.exp = cst_exp[tok];
      if (cst_flag[tok]) rc.flag = 1u;
    }
  }
  return rc;
}

// ------------------------------------------------------------------------------------------
// flow kernel for 17..64 operand rows on v_mfma_i32_32x32x32_i8 (4.0 POPS sustained where the
// 16x16x64 form stops at 3.0: at these row counts the decode kernel is limited by the matrix pipe and
// the vector work around it as much as by memory). Same stream and ring as tk_flow_kernel; what
// differs is the lane map and the row stride of the operand rows, which is the compile-time
// RS = 32 * RT2 (the prep kernels write that stride), so that every LDS read of a K block is one
// base register plus an immediate. Lane L = 32*kappa + 16*h + r. A wave walks S PAIRS of adjacent
// tiles; per position and plane it loads, from tile h of the pair, the 16-byte pieces g = kappa
// (load 0) and g = 2+kappa (load 1, 512 bytes further) of row r: dword j of load l is the B operand
// (32 weight rows x 32 k) of k step (l, j). The A operand of that step is piece (kb, j, 2*l + kappa)
// of operand row 32*rt2 + (L & 31); it is read one step ahead of its use, the first step of a K
// block during the last step of the block before (also across tiles: the operand rows of K block 0
// are the same for every tile). Accumulator register i of lane L is row 32*rt2 + 8*(i/4) + 4*kappa
// + i%4 of the column (h, r): four consecutive registers are four consecutive rows, as the
// epilogues expect, and the two halves of a wave store 32 adjacent columns. Row constants live in
// LDS behind the rows (16 row groups per lane are too many for registers): 1 KiB more LDS.
// ------------------------------------------------------------------------------------------

typedef int v16i __attribute__((ext_vector_type(16)));

// ZMAP (launches in which some plane carries a zero-chunk map; instantiated in a translation unit of its own so that
// the plain forms keep their code and register budgets): as in tk_flow_kernel, a request for a marked chunk goes to
// the plane's resident all-zero chunk -- the same bytes from the cache instead of from memory, same arithmetic, same
// bits. The two halves of a wave walk different tiles, so the look-up is per lane; map words behind the row constants.
// SWAP (int8 contract only): weights as the first operand of the matrix instruction, as in tk_flow_kernel -- accumulator
// register c of lane L is then channel 8*(c/4) + 4*kappa + c%4 of the pair's 32 for token 32*rt2 + (L & 31): four
// consecutive registers are four consecutive output channels of one token, written with one store.
// (Held to 128 registers -- four waves per SIMD, two eight-wave workgroups per CU at 64 KiB of rows -- the two-plane
// form on a ring of two spills 10..16 registers and the headline's batch 8 falls from 5.63 to 5.10 TB/s.)
template <int P, int RT2, int DR, bool TABLE, bool ZMAP = false, bool SWAP = false>
__global__ __launch_bounds__(512) void tk_flow32_kernel(const TkProblem single, const TkProblem *__restrict__ table,
                                                        const int *__restrict__ wg_prob) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const TkProblem &pr = TABLE ? table[wg_prob[blockIdx.x]] : *single_problem();
  constexpr int RS = 32 * RT2;           // row stride of the operand rows, in LDS and in pr.ap
  constexpr unsigned POS = RS * 256u;    // bytes of operand rows per K block
  static_assert((DR - 1) * POS + (14u * RS + 32u) * 16u < 65536u, "LDS offsets must fit the immediate");
  const int NW = (int)(blockDim.x >> 6);  // 4 or 8 waves
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r16 = lane & 15, h = (lane >> 4) & 1, kappa = lane >> 5;
  const int nb = pr.nb, R = pr.R, S = pr.run_tiles, n_tiles = pr.n_tiles;
  const TkHot hot = make_hot(pr);
  const uint8_t *codes[P];
  const float *scales[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    codes[p] = pr.codes[p];
    scales[p] = pr.scales[p];
  }
  constexpr int D = DR - 1;
  const int nbpad = (nb + DR - 1) / DR * DR;
  const int first = ((blockIdx.x - pr.group_begin) * NW + wave) * 2 * S;  // first tile of this wave
  const unsigned plane_last = (unsigned)n_tiles * (unsigned)nb - 1u;      // last chunk of the plane
  const unsigned skip = (unsigned)nb * 1024u;                             // the sibling tile of the pair
  const unsigned lane_piece = (unsigned)(kappa * 16 + r16) * 16u;         // piece g = kappa of row r
  unsigned roff = (unsigned)(first + h) * (unsigned)nb * 1024u + lane_piece - skip;
  const unsigned run_last = (unsigned)(first + (S - 1) * 2 + h) * (unsigned)nb + (unsigned)nb - 1u;
  const unsigned last_off = min(run_last, plane_last) * 1024u + lane_piece;

  // ZMAP: map words of the chunks this workgroup can ask for, staged below (see tk_flow_kernel)
  const uint32_t *lds_z = (const uint32_t *)(smem + (size_t)nb * POS + 1024);
  const unsigned zero_off = (unsigned)n_tiles * (unsigned)nb * 1024u + lane_piece;
  const unsigned wg_first = (unsigned)(blockIdx.x - pr.group_begin) * (unsigned)(NW * 2 * S);
  const unsigned zc0 = min(wg_first, (unsigned)n_tiles - 1u) * (unsigned)nb;
  const unsigned zc1 = min(wg_first + (unsigned)(NW * 2 * S), (unsigned)n_tiles) * (unsigned)nb;  // exclusive
  const unsigned zw0 = zc0 >> 5, zwords = ZMAP ? ((max(zc1, zc0 + 1u) - 1u) >> 5) - zw0 + 1u : 0u;
  uint4 ring[DR][P][2];
  auto request = [&](int slot, bool real, bool tile_start, bool use_map) {
    roff += tile_start ? skip : 0u;
    const unsigned off = min(roff, last_off);
#pragma unroll
    for (int p = 0; p < P; ++p) {
      unsigned o = off;
      if constexpr (ZMAP) {
        const unsigned chunk = off >> 10;  // (differs between the halves of the wave)
        uint32_t word;
        if (use_map) {
          const unsigned wi = (chunk >> 5) - zw0;
          word = wi < zwords ? lds_z[(unsigned)p * zwords + wi] : 0u;
        } else {  // the first requests of a workgroup, before its map words are in LDS: straight from memory
          const uint32_t *zm = pr.zmap[p];
          word = zm ? gload(zm + (chunk >> 5)) : 0u;
        }
        if ((word >> (chunk & 31u)) & 1u) o = zero_off + ((chunk & (unsigned)(TK_ZERO_CHUNKS - 1)) << 10);
      }
      ring[slot][p][0] = gload16_stream(codes[p] + (size_t)o);
      ring[slot][p][1] = gload16_stream(codes[p] + (size_t)o + 512);
    }
    roff += real ? 1024u : 0u;
  };
#pragma unroll
  for (int d = 0; d < D; ++d) request(d, d < nb, d == 0, false);

  // stage the operand rows of the problem in LDS (stride RS: the rows past R hold whatever the
  // workspace held, and feed accumulators that are never stored), and the row constants behind them
  uint8_t *cst = smem + (size_t)nb * POS;  // int rowsum[64] | float scale or int exponent [64] | uint flag[64]
  {
    const uint4 *ap4 = (const uint4 *)pr.ap;
    uint4 *lds4w = (uint4 *)smem;
    const int cnt = nb * 16 * RS;
    for (int idx = threadIdx.x; idx < cnt; idx += (int)blockDim.x) lds4w[idx] = gload16(ap4 + idx);
    if ((int)threadIdx.x < 64) {
      const int m = (int)threadIdx.x;
      int rsv = 0, ex = 0;
      float asv = 1.0f;
      unsigned fl = 0;
      if (m < R) rsv = gload(hot.rowsum + m);
      if (hot.mode == TK_MODE_INT8) {
        if (m < R && hot.act_scale) asv = gload(hot.act_scale + m);
        if (m < R && hot.flags) fl = gload(hot.flags + m);
        ((float *)(cst + 256))[m] = asv;
      } else {
        if (m < hot.M) {
          ex = gload(hot.exps + m);
          if (hot.flags) fl = gload(hot.flags + m);
        }
        ((int *)(cst + 256))[m] = ex;
      }
      ((int *)cst)[m] = rsv;
      ((uint32_t *)(cst + 512))[m] = fl;
    }
    if constexpr (ZMAP) {
      uint32_t *lz = (uint32_t *)(smem + (size_t)nb * POS + 1024);
      for (unsigned idx = threadIdx.x; idx < (unsigned)P * zwords; idx += blockDim.x) {
        const unsigned p = idx / zwords, w = idx - p * zwords;
        lz[idx] = pr.zmap[p] ? gload(pr.zmap[p] + zw0 + w) : 0u;
      }
    }
  }
  __syncthreads();
  // does any row of the problem take the exact fallback?
  unsigned any_flag = 0;
  if (hot.flags) {
    const uint32_t *cf = (const uint32_t *)(cst + 512);
    const int lim = hot.mode == TK_MODE_INT8 ? R : hot.M;
    for (int m = 0; m < lim; ++m) any_flag |= cf[m];
  }

  // A operand of k step (l, j) = step 4*l + j of the K block whose rows start at byte `base`
  const unsigned abase0 = (unsigned)(kappa * RS + (lane & 31)) * 16u;
  auto lds_a = [&](unsigned base, int step, int rt2) -> v4i {
    const int l = step >> 2, j = step & 3;
    return *(const v4i *)(smem + base + (unsigned)(((j * 4 + 2 * l) * RS + rt2 * 32) * 16));
  };
  v4i a_cur[RT2];
#pragma unroll
  for (int rt2 = 0; rt2 < RT2; ++rt2) a_cur[rt2] = lds_a(abase0, 0, rt2);

  for (int s = 0; s < S; ++s) {
    const int t = first + 2 * s + h;  // this lane's tile of the pair
    float sc[P];
    float sc4[SWAP ? P : 1][SWAP ? 4 : 1][4];  // SWAP: the scales of this lane's sixteen channels of the pair
    if constexpr (SWAP) {
      const int c0 = (first + 2 * s) * 16 + 4 * kappa;
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) sc4[p][q][r] = gload(scales[p] + min(c0 + 8 * q + r, hot.n - 1));
    } else {
      const int n = min(t * 16 + r16, hot.n - 1);
#pragma unroll
      for (int p = 0; p < P; ++p) sc[p] = gload(scales[p] + n);
    }
    v16i acc[RT2][P];
#pragma unroll
    for (int rt2 = 0; rt2 < RT2; ++rt2)
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int c = 0; c < 16; ++c) acc[rt2][p][c] = 0;

    int kbg = 0;
    do {
      const unsigned gbase = abase0 + (unsigned)kbg * POS;
#pragma unroll
      for (int d = 0; d < DR; ++d) {
        const int kb = kbg + d;
        {
          int kb2 = kb + D;
          if (kb2 >= nbpad) kb2 -= nbpad;
          request((d + D) % DR, kb2 < nb, kb2 == 0, true);
        }
        if (kb < nb) {
          const unsigned base = gbase + (unsigned)d * POS;
          const unsigned nbase = kb + 1 < nb ? base + POS : abase0;  // K block 0 of the next tile
#pragma unroll
          for (int step = 0; step < 8; ++step) {
            v4i a_nxt[RT2];
#pragma unroll
            for (int rt2 = 0; rt2 < RT2; ++rt2) a_nxt[rt2] = step < 7 ? lds_a(base, step + 1, rt2) : lds_a(nbase, 0, rt2);
#pragma unroll
            for (int p = 0; p < P; ++p) {
              const uint4 w = ring[d][p][step >> 2];
              const int j = step & 3;
              const uint32_t wj = j == 0 ? w.x : (j == 1 ? w.y : (j == 2 ? w.z : w.w));
              const v4i b = expand_codes(wj);
#pragma unroll
              for (int rt2 = 0; rt2 < RT2; ++rt2)
                acc[rt2][p] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a_cur[rt2], acc[rt2][p], 0, 0, 0)
                                   : __builtin_amdgcn_mfma_i32_32x32x32_i8(a_cur[rt2], b, acc[rt2][p], 0, 0, 0);
            }
#pragma unroll
            for (int rt2 = 0; rt2 < RT2; ++rt2) a_cur[rt2] = a_nxt[rt2];
          }
        }
      }
      kbg += DR;
    } while (kbg < nbpad);

    if constexpr (SWAP) {
      const int c0 = (first + 2 * s) * 16 + 4 * kappa;
      const int *cst_rs = (const int *)cst;
      const float *cst_as = (const float *)(cst + 256);
      const uint32_t *cst_fl = (const uint32_t *)(cst + 512);
#pragma unroll
      for (int rt2 = 0; rt2 < RT2; ++rt2) {
        const int m = rt2 * 32 + (lane & 31);
        if (m >= R) continue;
        const int rs = cst_rs[m];
        const float as = cst_as[m];
        const unsigned fl = cst_fl[m];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n0 = c0 + 8 * q;
          if (n0 >= hot.n) continue;
          v4i av[P];
          float sq[P][4];
#pragma unroll
          for (int p = 0; p < P; ++p) {
            av[p] = v4i{acc[rt2][p][4 * q], acc[rt2][p][4 * q + 1], acc[rt2][p][4 * q + 2], acc[rt2][p][4 * q + 3]};
#pragma unroll
            for (int r = 0; r < 4; ++r) sq[p][r] = sc4[p][q][r];
          }
          flow_epilogue_swapped<P>(hot, pr, m, n0, av, sq, rs, as, fl);
        }
      }
      continue;
    }
    const int n = t * 16 + r16;
    if (t < n_tiles && n < hot.n) {
#pragma unroll
      for (int rt2 = 0; rt2 < RT2; ++rt2)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rl = rt2 * 32 + 8 * q + 4 * kappa;
          const RowConst rc = row_const_from_lds(cst, hot.mode, R, hot.M, rl);
          v4i av[P];
#pragma unroll
          for (int p = 0; p < P; ++p) av[p] = v4i{acc[rt2][p][4 * q], acc[rt2][p][4 * q + 1], acc[rt2][p][4 * q + 2], acc[rt2][p][4 * q + 3]};
          flow_epilogue<P>(hot, n, rl, av, sc, rc);
        }
      if (any_flag) {
        for (int rt2 = 0; rt2 < RT2; ++rt2)
          for (int q = 0; q < 4; ++q) {
            const int rowbase = rt2 * 32 + 8 * q + 4 * kappa;
            const unsigned fl = row_flags(pr, rowbase);
            if (fl) exact_rows(pr, n, rowbase, fl);
          }
      }
    }
  }
}

template <typename K>
static hipError_t flow_launch_one(K kernel, hipStream_t s, const TkProblem &sg, const TkProblem *table,
                                  const int *wg_prob, const TkLaunchCfg &cfg, int threads) {
  if (cfg.lds_bytes > 64 * 1024) {
    hipError_t e = tk_raise_lds_limit((const void *)kernel, 160 * 1024);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, dim3(cfg.grid), dim3(threads), cfg.lds_bytes, s, sg, table, wg_prob);
  return hipGetLastError();
}

