// gfx950 decode GEMV that streams base-3 packed weights (five trits per byte, 1.625 bits per trit
// where the 2-bit layout spends 2) and unpacks them in the kernel.
//
// The byte code is TQ1_0's (crates/tritium-format/src/tq1.rs:18-30): a byte holds v = sum d_n * 3^(4-n)
// over the codes d_n = trit + 1 as ceil(v * 256 / 243), and digit n comes back as
// ((uint8)(byte * 3^n) * 3) >> 8 -- the decode the reference's own base-3 GEMV runs per element
// (crates/tritium-cuda/kernels/tq2_0_add.cu:744-774). What differs from a TQ1_0 row is only which
// trit sits in which digit of which byte: the stream is cut for the int8 MFMA this library contracts
// with (chunks of 16 rows x 256 k, 13 bytes per lane; layout in tk_internal.h), so that
//   * digits 1..4 of a byte are the four int8 codes of one operand dword: one LDS read from a table of
//     256 entries, replicated per lane so that the 64 lanes of a wave never meet in a bank (the read
//     address is one v_perm_b32: [lane*4 | byte << 8]);
//   * digit 0 of the four bytes of a dword is a fifth operand dword: ((b * 3) >> 8) on the even and
//     the odd bytes, two multiplies by three.
// Per 256 trits of 16 rows a wave issues 13 table reads and about 40 vector instructions in place of
// the 32 shift-and pairs of the 2-bit layout, and loads 832 bytes in place of 1024.
//
// Everything else -- operand rows resident in LDS, runs of output tiles walked with a ring of
// prefetches, the epilogues and the reference-order fallback -- is the flow kernel's (tk_kernels.hip).
// The accumulators are the same integers, so the outputs carry the same bits.

#include "tk_device.h"

// ------------------------------------------------------------------------------------------
// re-encode a T16 plane (1 KiB chunks of 2-bit codes) into the base-3 stream (832-byte chunks)
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(TK_WG) void tk_encode_base3_kernel(const uint8_t *__restrict__ codes,
                                                                uint8_t *__restrict__ codes3, size_t chunks) {
  const size_t idx = (size_t)blockIdx.x * TK_WG + threadIdx.x;
  const size_t chunk = idx >> 6;
  const unsigned lane = (unsigned)(idx & 63);
  if (chunk >= chunks) return;
  const uint4 w = gload16(codes + chunk * TK_CHUNK_BYTES + lane * 16);
  const uint32_t wj[4] = {w.x, w.y, w.z, w.w};
  auto code = [&](int j, int s, int b) -> unsigned {
    const unsigned c = (wj[j] >> (8 * b + 2 * s)) & 3u;
    return c > 2u ? 2u : c;  // (the reserved code never passes the upload checks)
  };
  auto enc = [](unsigned d0, unsigned d1, unsigned d2, unsigned d3, unsigned d4) -> unsigned {
    const unsigned v = (((d0 * 3 + d1) * 3 + d2) * 3 + d3) * 3 + d4;
    return (v * 256u + 242u) / 243u;
  };
  uint32_t q[3] = {0, 0, 0};
#pragma unroll
  for (int t = 0; t < 12; ++t) {
    const unsigned byte = enc(code(t / 4, 3, t % 4), code(t / 3, t % 3, 0), code(t / 3, t % 3, 1), code(t / 3, t % 3, 2),
                              code(t / 3, t % 3, 3));
    q[t / 4] |= byte << (8 * (t % 4));
  }
  const unsigned last = enc(0, code(3, 3, 0), code(3, 3, 1), code(3, 3, 2), code(3, 3, 3));
  uint8_t *dst = codes3 + chunk * TK_B3_CHUNK_BYTES;
  uint32_t *dq = (uint32_t *)(dst + lane * 12);
  gstore(dq + 0, q[0]);
  gstore(dq + 1, q[1]);
  gstore(dq + 2, q[2]);
  gstore(dst + 768 + lane, (uint8_t)last);
}

hipError_t tk_launch_encode_base3(hipStream_t s, const uint8_t *codes, uint8_t *codes3, size_t chunks) {
  if (!chunks) return hipSuccess;
  const size_t threads = chunks * 64;
  hipLaunchKernelGGL(tk_encode_base3_kernel, dim3((unsigned)((threads + TK_WG - 1) / TK_WG)), dim3(TK_WG), 0, s, codes,
                     codes3, chunks);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// the flow kernel over the base-3 stream
// ------------------------------------------------------------------------------------------

// A lane's 13 bytes of one chunk: three dwords and the last byte, zero-extended.
typedef unsigned tk_v3u __attribute__((ext_vector_type(3)));
typedef tk_v3u tk_v3u_a4 __attribute__((aligned(4)));  // twelve bytes at a 4-byte boundary: one global_load_dwordx3
struct TkB3Piece {
  uint32_t q[3];
  uint32_t h;
};

#define TK_LDS __attribute__((address_space(3)))

// digits 1..4 of byte k of w, as four int8 codes: the table entry of that byte in this lane's bank
// (the table starts at LDS address 0: the kernel has no static LDS in front of its dynamic array, which the
// build verifies from the kernel's metadata: check_isa.NO_STATIC_LDS)
__device__ __forceinline__ int b3_table(uint32_t w, uint32_t lane4, int k) {
  // v_perm_b32: selector bytes 0..3 pick from the second operand, 4..7 from the first, 0x0c is zero
  const uint32_t addr = __builtin_amdgcn_perm(w, lane4, 0x0C0C0400u | ((uint32_t)k << 8));
  return *(const TK_LDS int *)(uintptr_t)addr;
}

// digit 0 of the four bytes of w: (b * 3) >> 8 per byte
__device__ __forceinline__ int b3_first_digits(uint32_t w) {
  const uint32_t te = (w & 0x00FF00FFu) * 3u;
  const uint32_t to = ((w >> 8) & 0x00FF00FFu) * 3u;
  return (int)(((te >> 8) & 0x00030003u) | (to & 0x03000300u));
}

// Eight waves per workgroup; with one row tile of short rows two workgroups (two tables) share a CU:
// four waves per SIMD, 128 registers. Bytes in flight decide this kernel's rate as they do the 2-bit
// kernel's: measured, a variant that issues each position's LDS reads one MFMA step ahead needs ~150
// registers (three waves per SIMD as one twelve-wave workgroup) and is 4-15% slower than this one.
#define TK_B3_WAVES 8
template <int P, int RT, int TW, bool TABLE>
__global__ __launch_bounds__(TK_B3_WAVES * 64) void tk_flow3_kernel(const TkProblem single, const TkProblem *__restrict__ table,
                                                       const int *__restrict__ wg_prob) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // the decode table, then the operand rows
  const TkProblem &pr = TABLE ? table[wg_prob[blockIdx.x]] : *single_problem();
  const int NW = (int)(blockDim.x >> 6);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int i = lane & 15, g = lane >> 4;
  const int nb = pr.nb, R = pr.R, S = pr.run_tiles, n_tiles = pr.n_tiles;
  const TkHot hot = make_hot(pr);
  const uint8_t *codes[P];
  const float *scales[P];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    codes[p] = pr.codes3[p];
    scales[p] = pr.scales[p];
  }
  // The stream of a run is walked exactly as the 2-bit flow kernel walks its own: positions
  // q = s*nbpad + kb with nbpad = nb rounded up to the ring size, at every position (padding included)
  // the chunks D positions ahead are requested into the slot consumed one position ago, requests past
  // the end of a run ask again for its last chunk. Only the chunk size differs.
  constexpr int DR = 4, D = DR - 1;
  constexpr unsigned CB = TK_B3_CHUNK_BYTES;
  const int nbpad = (nb + DR - 1) / DR * DR;
  const int first = ((blockIdx.x - pr.group_begin) * NW + wave) * TW * S;
  const unsigned plane_last = (unsigned)n_tiles * (unsigned)nb - 1u;
  const unsigned skip = (unsigned)(TW - 1) * (unsigned)nb * CB;
  unsigned roff[TW], last_off[TW];  // byte offsets of chunks inside a plane
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    roff[tw] = (unsigned)(first + tw) * (unsigned)nb * CB - skip;
    const unsigned run_last = (unsigned)(first + (S - 1) * TW + tw) * (unsigned)nb + (unsigned)nb - 1u;
    last_off[tw] = min(run_last, plane_last) * CB;
  }
  const unsigned lane12 = (unsigned)lane * 12u, lane_h = 768u + (unsigned)lane;
  TkB3Piece ring[DR][TW][P];
  auto request = [&](int slot, bool real, bool tile_start) {
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      roff[tw] += tile_start ? skip : 0u;
      const unsigned off = min(roff[tw], last_off[tw]);
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const uint8_t *base = codes[p] + (size_t)off;
        // (non-temporal, like the 2-bit stream: every byte is read once per launch)
#if TK_STREAM_NT
        const tk_v3u d = __builtin_nontemporal_load((const TK_GLOBAL tk_v3u_a4 *)(base + lane12));
        const uint8_t hb = __builtin_nontemporal_load((const TK_GLOBAL uint8_t *)(base + lane_h));
#else
        const tk_v3u d = *(const TK_GLOBAL tk_v3u_a4 *)(base + lane12);
        const uint8_t hb = *(const TK_GLOBAL uint8_t *)(base + lane_h);
#endif
        ring[slot][tw][p].q[0] = d.x;
        ring[slot][tw][p].q[1] = d.y;
        ring[slot][tw][p].q[2] = d.z;
        ring[slot][tw][p].h = (uint32_t)hb;
      }
      roff[tw] += real ? CB : 0u;
    }
  };
#pragma unroll
  for (int d = 0; d < D; ++d) request(d, d < nb, d == 0);

  // the decode table: entry b (digits 1..4 of byte b as four int8 codes), one copy per lane
  {
    uint32_t *tab = (uint32_t *)smem;
    for (int idx = threadIdx.x; idx < TK_B3_TABLE_BYTES / 4; idx += (int)blockDim.x) {
      unsigned q = ((unsigned)(idx >> 6) * 3u) & 0xFFu;  // past digit 0
      uint32_t v = 0;
#pragma unroll
      for (int n = 0; n < 4; ++n) {
        const unsigned t = q * 3u;
        v |= (t >> 8) << (8 * n);
        q = t & 0xFFu;
      }
      tab[idx] = v;
    }
  }
  // every operand row of the problem behind it
  uint8_t *rows = smem + TK_B3_TABLE_BYTES;
  {
    const uint4 *ap4 = (const uint4 *)pr.ap;
    uint4 *lds4w = (uint4 *)rows;
    const int cnt = nb * 16 * R;
    for (int idx = threadIdx.x; idx < cnt; idx += (int)blockDim.x) lds4w[idx] = gload16(ap4 + idx);
  }
  RowConst rc[RT];
  unsigned any_flag = 0;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    rc[rt] = load_row_const(hot, rt * 16 + 4 * g);
    any_flag |= rc[rt].flag;
  }
  __syncthreads();
  const uint4 *lds4 = (const uint4 *)rows;
  int arow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) arow[rt] = min(rt * 16 + i, R - 1);
  const uint32_t lane4 = (uint32_t)lane * 4u;

  for (int s = 0; s < S; ++s) {
    float sc[TW][P];
#pragma unroll
    for (int tw = 0; tw < TW; ++tw) {
      const int n = min((first + s * TW + tw) * 16 + i, hot.n - 1);
#pragma unroll
      for (int p = 0; p < P; ++p) sc[tw][p] = gload(scales[p] + n);
    }
    v4i acc[TW][RT][P];
#pragma unroll
    for (int tw = 0; tw < TW; ++tw)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int p = 0; p < P; ++p) acc[tw][rt][p] = v4i{0, 0, 0, 0};

    int kbg = 0;
    do {
#pragma unroll
      for (int d = 0; d < DR; ++d) {
        const int kb = kbg + d;
        {
          int kb2 = kb + D;
          if (kb2 >= nbpad) kb2 -= nbpad;
          request((d + D) % DR, kb2 < nb, kb2 == 0);
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
                const TkB3Piece &w = ring[d][tw][p];
                v4i b;
                // bytes 3j, 3j+1, 3j+2 of the twelve: dword t/4, byte t%4
                b.x = b3_table(w.q[(3 * j) / 4], lane4, (3 * j) % 4);
                b.y = b3_table(w.q[(3 * j + 1) / 4], lane4, (3 * j + 1) % 4);
                b.z = b3_table(w.q[(3 * j + 2) / 4], lane4, (3 * j + 2) % 4);
                b.w = j < 3 ? b3_first_digits(w.q[j < 3 ? j : 0]) : b3_table(w.h, lane4, 0);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                  acc[tw][rt][p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[rt], b, acc[tw][rt][p], 0, 0, 0);
              }
          }
        }
      }
      kbg += DR;
    } while (kbg < nbpad);

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
          const unsigned fl = row_flags(pr, rowbase);
          if (fl) exact_rows(pr, n, rowbase, fl);  // reads the plane's 2-bit copy
        }
      }
    }
  }
}

// runs per wave: two for one plane (as the 2-bit kernel keeps two there), one otherwise
int tk_flow3_runs_per_wave(int planes) { return planes == 1 ? 2 : 1; }
int tk_flow3_waves(int rt) { (void)rt; return TK_B3_WAVES; }

template <typename K>
static hipError_t flow3_launch_one(K kernel, hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                   const TkLaunchCfg &cfg) {
  // the table alone is 64 KiB: the dynamic LDS limit has to be raised
  hipError_t e = tk_raise_lds_limit((const void *)kernel, 160 * 1024);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kernel, dim3(cfg.grid), dim3(cfg.waves * 64), cfg.lds_bytes, s, sg, table, wg_prob);
  return hipGetLastError();
}

template <int P, int RT>
static hipError_t launch_flow3_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                  const TkLaunchCfg &cfg) {
  constexpr int TW = P == 1 ? 2 : 1;
  if (table) return flow3_launch_one(tk_flow3_kernel<P, RT, TW, true>, s, sg, table, wg_prob, cfg);
  return flow3_launch_one(tk_flow3_kernel<P, RT, TW, false>, s, sg, table, wg_prob, cfg);
}

hipError_t tk_launch_flow3(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                           const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  if (cfg.rt != 1 && cfg.rt != 2) return hipErrorInvalidValue;
  switch (cfg.planes) {
    case 1: return cfg.rt == 1 ? launch_flow3_pr<1, 1>(s, sg, table, wg_prob, cfg) : launch_flow3_pr<1, 2>(s, sg, table, wg_prob, cfg);
    case 2: return cfg.rt == 1 ? launch_flow3_pr<2, 1>(s, sg, table, wg_prob, cfg) : launch_flow3_pr<2, 2>(s, sg, table, wg_prob, cfg);
    case 3: return cfg.rt == 1 ? launch_flow3_pr<3, 1>(s, sg, table, wg_prob, cfg) : launch_flow3_pr<3, 2>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}
