// gfx950 prefill GEMM, 256 x 224 outputs per workgroup, one plane, int8 contract: the weight tile is expanded
// from 2-bit codes to int8 ONCE per workgroup, into LDS, and every wave reads finished operands from there.
//
// In the other prefill kernels every wave expands the codes of its own columns in registers, seven vector
// instructions per matrix operand that two matrix instructions use: the expansion occupies the SIMD about as
// long as the matrix pipe, and the two do not overlap well. Here a workgroup is 256 operand rows x 14 weight
// tiles (224 outputs). Its waves split the ROWS (a wave owns 64 or 32 rows and all 224 outputs), so
//  * the int8 form of the weight tile is shared by all of them: per K block (256 k) the waves expand the 14
//    one-KiB chunks between them (a chunk per wave and round) and write 56 KiB of operands to LDS, double
//    buffered, one barrier per K block -- under one vector instruction per matrix instruction;
//  * a wave's activation operands are its own, so they skip LDS: 16-byte pieces go straight from the operand
//    rows in L2 to registers, four k steps ahead (a ring of four register sets, waits by hand);
//  * per k step (32 k) a wave reads 7 weight operands from LDS for 14 (or 7) matrix instructions.
// Same codes, same integers, same epilogue arithmetic as every other kernel: identical bits.
//
// LDS operand order: a K block has 8 k steps t = 2j + l (j = dword of a lane's 16-byte piece, l = half of the
// block); operand (t, p) of pair p (two adjacent tiles, 32 outputs) is one KiB at ((t * 7 + p) * 1024), lane
// L = 32 kappa + 16 h + r holds the 16 codes of slot order of row r of tile 2p + h, piece g = 2l + kappa --
// what expand_codes() makes of dword j of the T16 chunk's lane (g, r). The activation operand of k step t is
// the pair of segments (4j + 2l + kappa) = 2t + kappa of the operand rows.
//
// Takes what the 128-row kernel takes: one plane, int8 operand rows, f32 or bf16 output rows of whole 16-byte
// pieces at a 16-byte aligned address, no residual.

#include <type_traits>

#include "tk_device.h"

typedef int v16i_x __attribute__((ext_vector_type(16)));

#define TK_G256_PAIRS 7                           // pairs of tiles (32 outputs each) of a full column block
#define TK_G256_TILES 14
#define TK_G256_BBUF(pw) ((pw) * 8 * 1024)        // the int8 weight operands of one K block of pw pairs
#define TK_G256_PD 3                              // LDS reads in flight ahead of the matrix instructions
#define TK_G256_FIRST 4                           // k step of a K block in which the expansion rounds begin
#define TK_G256_STAGE 16896                       // epilogue staging per wave: 32 tokens x (224 bf16 or 128 f32, + 16 bytes)
#define TK_G256_WAVE_LDS TK_G256_STAGE


template <int I, int N, typename F>
__device__ __forceinline__ void tk_static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    tk_static_for<I + 1, N>(f);
  }
}

// LDS operations issued after the read of operand q (= 7 t + p) and before the wait in front of its matrix
// instructions: the next reads (PD of them while the block has that many left) and, behind pair 3 (the last pair
// of a block of three) of the k steps FIRST .. FIRST + NR - 1, the four writes of an expansion round.
template <int NR, int PW>
__host__ __device__ constexpr int tk_g256_younger(int q) {
  int n = 8 * PW - 1 - q < TK_G256_PD ? 8 * PW - 1 - q : TK_G256_PD;
  for (int r = 0; r < NR; ++r) {
    const int qw = (TK_G256_FIRST + r) * PW + (PW > 3 ? 3 : PW - 1);
    if (qw < q && q <= qw + TK_G256_PD) n += 4;
  }
  return n;
}

// One workgroup: 256 operand rows (row block bm) x PW pairs of weight tiles starting at tile0.
// RT2 = 2: four waves of 64 rows; RT2 = 1: eight waves of 32 rows.
template <int RT2, int PW>
__device__ __forceinline__ void tk_g256_body(const TkProblem &pr, const TkHot &hot, uint8_t *smem, int bm, int tile0) {
  constexpr int NW = 8 / RT2, WROWS = 32 * RT2, NT = 2 * PW, Q = 8 * PW;
  constexpr int NR = (NT + NW - 1) / NW;  // expansion rounds per K block
  constexpr int PD = TK_G256_PD, FIRST = TK_G256_FIRST, WP = PW > 3 ? 3 : PW - 1;
  static_assert(FIRST + NR <= 8, "the expansion rounds fit behind the k step that waits for the codes");
  const int tid = (int)threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r16 = lane & 15, r32 = lane & 31, kappa = lane >> 5, g = lane >> 4;
  const int nb = pr.nb, R = pr.R, n_tiles = pr.n_tiles, rs = pr.rs;
  const uint8_t *codes = pr.codes[0];
  const uint8_t *ap8 = (const uint8_t *)pr.ap;
  const int row_base = bm * 256 + wave * WROWS;

  // ---- operand addresses ----
  // activation piece of (K block kb, k step t, 32-row tile rt2): ap + ((kb*16 + 2t + kappa) * rs + row) * 16
  unsigned a_off[RT2];
#pragma unroll
  for (int rt2 = 0; rt2 < RT2; ++rt2)
    a_off[rt2] = (unsigned)(((size_t)kappa * (size_t)rs + (size_t)min(row_base + rt2 * 32 + r32, R - 1)) * 16);
  const size_t a_step = (size_t)rs * 32, a_block = (size_t)rs * 256;
  // this wave's chunk of expansion round r: c = r * NW + wave (past the last: the last again, the same bytes to the same place)
  unsigned c_off[NR], w_lane[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int c = min(r * NW + wave, NT - 1);
    const int tile = min(tile0 + c, n_tiles - 1);
    c_off[r] = (unsigned)((size_t)tile * (size_t)nb * 1024 + (size_t)lane * 16);
    // lane (g, r16) of tile c = 2p + h holds piece g = 2l + kappa': operand (t = 2j + l, p), lane 32 kappa' + 16 h + r16
    w_lane[r] = (unsigned)(((g >> 1) * PW + (c >> 1)) * 1024 + (32 * (g & 1) + 16 * (c & 1) + r16) * 16);
  }
  const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) uint8_t *)smem;
  const unsigned rd_lane[2] = {lds0 + (unsigned)lane * 16u, lds0 + (unsigned)TK_G256_BBUF(PW) + (unsigned)lane * 16u};

  auto load_a = [&](v4i (&dst)[RT2], int kb, int t) {
    const uint8_t *base = ap8 + (size_t)min(kb, nb - 1) * a_block + (size_t)t * a_step;  // wave-uniform
#pragma unroll
    for (int rt2 = 0; rt2 < RT2; ++rt2)
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst[rt2]) : "v"(a_off[rt2]), "s"(base));
  };
  auto load_codes = [&](v4i (&cs)[NR], int kb) {
    const uint8_t *base = codes + (size_t)min(kb, nb - 1) * 1024;  // wave-uniform
#pragma unroll
    for (int r = 0; r < NR; ++r) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(cs[r]) : "v"(c_off[r]), "s"(base));
  };
  // one expansion round: the chunk's four dwords become four operands of the same pair (k steps 2j + l)
  auto expand_round = [&](const v4i &cw, unsigned waddr) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const v4i e = expand_codes((uint32_t)cw[j]);
      asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(waddr), "v"(e), "n"(j * 2 * PW * 1024));
    }
  };
  auto lds_read = [&](v4i &b, unsigned addr, auto off_c) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b) : "v"(addr), "n"(decltype(off_c)::value));
  };

  // D[i][j] of the matrix instruction has i = token of the 32-row tile and j = output column of the pair: lane
  // (kappa, r32) holds column r32 and, in register 4q + r, token 8q + 4 kappa + r. The activation operand goes first
  // (measured on this kernel: with the operand that comes fresh from LDS as the first source the loop is 13% slower).
  // The codes are trit + 1, so sum(code * a) = sum(trit * a) + rowsum: the accumulators start at -rowsum of their token.
  v16i_x acc[RT2][PW];
#pragma unroll
  for (int rt2 = 0; rt2 < RT2; ++rt2) {
    const int tok0 = row_base + rt2 * 32;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int neg[4];
      if (tok0 + 32 <= R) {
        const v4i r4 = *(const TK_GLOBAL v4i *)(hot.rowsum + tok0 + 8 * q + 4 * kappa);
        neg[0] = -r4.x; neg[1] = -r4.y; neg[2] = -r4.z; neg[3] = -r4.w;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) neg[r] = -gload(hot.rowsum + min(tok0 + 8 * q + 4 * kappa + r, R - 1));
      }
#pragma unroll
      for (int p = 0; p < PW; ++p)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[rt2][p][4 * q + r] = neg[r];
    }
  }

  v4i a[4][RT2], b[4], cset[NR];

  // ---- prologue: K block 0 expanded into buffer 0, the first four k steps of activations on their way ----
  load_codes(cset, 0);
#pragma unroll
  for (int t = 0; t < 4; ++t) load_a(a[t], 0, t);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * RT2));  // the codes have landed
#pragma unroll
  for (int r = 0; r < NR; ++r) asm volatile("" : "+v"(cset[r]));
#pragma unroll
  for (int r = 0; r < NR; ++r) expand_round(cset[r], lds0 + w_lane[r]);
  asm volatile("s_waitcnt lgkmcnt(0)");
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int q = 0; q < PD; ++q) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[q]) : "v"(rd_lane[0]), "n"(q * 1024));

  // ---- one K block: buffer `cur` is read, the codes of block kb + 1 are loaded and expanded into the other ----
  auto block = [&](auto cur_c, int kb) {
    constexpr int cur = decltype(cur_c)::value;
    load_codes(cset, kb + 1);
    tk_static_for<0, Q>([&](auto q_c) {
      constexpr int q = decltype(q_c)::value, t = q / PW, p = q % PW;
      if constexpr (p == 0) {
        // the activation pieces of k step t have landed; younger: three k steps, and until step 4 the codes
        if constexpr (t < 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * RT2 + NR));
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * RT2));
#pragma unroll
        for (int rt2 = 0; rt2 < RT2; ++rt2) asm volatile("" : "+v"(a[t % 4][rt2]));
        if constexpr (t == FIRST) {
#pragma unroll
          for (int r = 0; r < NR; ++r) asm volatile("" : "+v"(cset[r]));
        }
      }
      if constexpr (q + PD < Q) lds_read(b[(q + PD) % 4], rd_lane[cur], std::integral_constant<int, (q + PD) * 1024>{});
      asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(tk_g256_younger<NR, PW>(q)));
      asm volatile("" : "+v"(b[q % 4]));
#pragma unroll
      for (int rt2 = 0; rt2 < RT2; ++rt2)
                acc[rt2][p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t % 4][rt2], b[q % 4], acc[rt2][p], 0, 0, 0);
      if constexpr (p == WP && t >= FIRST && t - FIRST < NR) expand_round(cset[t - FIRST], rd_lane[cur ^ 1] - (unsigned)lane * 16u + w_lane[t - FIRST]);
      if constexpr (p == PW - 1) load_a(a[t % 4], t < 4 ? kb : kb + 1, (t + 4) % 8);  // into the set this step just used
    });
    asm volatile("s_waitcnt lgkmcnt(0)");  // this wave's operands of block kb + 1 are in LDS
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int q = 0; q < PD; ++q)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[q]) : "v"(rd_lane[cur ^ 1]), "n"(q * 1024));
  };
  int kb = 0;
  for (; kb + 2 <= nb; kb += 2) {
    block(std::integral_constant<int, 0>{}, kb);
    block(std::integral_constant<int, 1>{}, kb + 1);
  }
  if (kb < nb) block(std::integral_constant<int, 0>{}, kb);
  // the loads and reads issued for a block that does not exist must land before their registers are reused
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)");
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int rt2 = 0; rt2 < RT2; ++rt2) asm volatile("" : "+v"(a[t][rt2]));
#pragma unroll
  for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(b[q]));
#pragma unroll
  for (int r = 0; r < NR; ++r) asm volatile("" : "+v"(cset[r]));

  // ---- epilogue: out[m,n] = ((float)acc * scale[n]) * act_scale[m] (the accumulators started at -rowsum[m]): three
  //      vector instructions per output and half a conversion; the values are staged in this wave's own piece of LDS
  //      (free behind the loop's last barrier) and leave as two whole row segments per store instruction, 16 bytes
  //      per lane. ----
  unsigned my_flag = 0;
  if (hot.flags && tid < 256 && bm * 256 + tid < R) my_flag = gload(hot.flags + bm * 256 + tid) ? 1u : 0u;
  const int wg_flag = __syncthreads_or((int)my_flag);
  uint8_t *wl = smem + (size_t)wave * TK_G256_WAVE_LDS;
  const int col0 = tile0 * 16;
  float sc[PW];
#pragma unroll
  for (int p = 0; p < PW; ++p) sc[p] = gload(pr.scales[0] + min(col0 + p * 32 + r32, hot.n - 1));
  const int half = lane >> 5, piece = lane & 31;
  auto finish = [&](auto esz_c) {
    constexpr int ESZ = decltype(esz_c)::value;
    constexpr int NPASS = (ESZ == 2 || PW <= 4) ? 1 : 2;  // f32 rows of more than four pairs are staged in two column groups
#pragma unroll
    for (int rt2 = 0; rt2 < RT2; ++rt2) {
      const int tok0 = row_base + rt2 * 32;
      const bool plain = tok0 + 32 <= R && !wg_flag;  // no row of this tile needs a test
      float as[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (!hot.act_scale) {
#pragma unroll
          for (int r = 0; r < 4; ++r) as[4 * q + r] = 1.0f;
        } else if (tok0 + 32 <= R) {
          const v4u a4 = *(const TK_GLOBAL v4u *)(hot.act_scale + tok0 + 8 * q + 4 * kappa);
          as[4 * q] = __uint_as_float(a4.x); as[4 * q + 1] = __uint_as_float(a4.y);
          as[4 * q + 2] = __uint_as_float(a4.z); as[4 * q + 3] = __uint_as_float(a4.w);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) as[4 * q + r] = gload(hot.act_scale + min(tok0 + 8 * q + 4 * kappa + r, R - 1));
        }
      }
      tk_static_for<0, NPASS>([&](auto ps_c) {
        constexpr int ps = decltype(ps_c)::value;
        constexpr int p0 = ps == 0 ? 0 : 4, p1 = (NPASS == 1 || ps == 1) ? PW : 4;
        constexpr int NCOL = (p1 - p0) * 32, STRIDE = NCOL * ESZ + 16, PPR = NCOL * ESZ / 16;
        static_assert(32 * STRIDE <= TK_G256_STAGE && STRIDE % 16 == 0 && PPR <= 32, "a pass fits the wave's staging area");
        uint8_t *lane_base = wl + (size_t)(4 * kappa) * STRIDE + (size_t)r32 * ESZ;
#pragma unroll
        for (int p = p0; p < p1; ++p)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float f[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) f[r] = __fmul_rn(__fmul_rn((float)acc[rt2][p][4 * q + r], sc[p]), as[4 * q + r]);
            uint8_t *dst = lane_base + (size_t)(8 * q) * STRIDE + (size_t)(p - p0) * 32 * ESZ;
            if (ESZ == 2) {
              const uint32_t d01 = f32x2_to_bf16x2(f[0], f[1]), d23 = f32x2_to_bf16x2(f[2], f[3]);
              *(uint16_t *)dst = (uint16_t)d01;
              *(uint16_t *)(dst + STRIDE) = (uint16_t)(d01 >> 16);
              *(uint16_t *)(dst + 2 * STRIDE) = (uint16_t)d23;
              *(uint16_t *)(dst + 3 * STRIDE) = (uint16_t)(d23 >> 16);
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r) *(float *)(dst + r * STRIDE) = f[r];
            }
          }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // lanes 0..PPR-1 carry the pieces of an even staged row, lanes 32..32+PPR-1 those of the odd row behind it
        const int c = col0 + p0 * 32 + piece * (16 / ESZ);
        if (piece < PPR && c < hot.n) {
          uint8_t *gp = (uint8_t *)hot.out + ((size_t)(tok0 + half) * (size_t)hot.n + (size_t)c) * ESZ;
          const uint8_t *sp = wl + (size_t)half * STRIDE + (size_t)piece * 16;
          const size_t gstep = (size_t)hot.n * ESZ * 2;
          if (plain) {
#pragma unroll
            for (int it = 0; it < 16; ++it) *(TK_GLOBAL v4u *)(gp + it * gstep) = *(const v4u *)(sp + it * 2 * STRIDE);
          } else {
            for (int it = 0; it < 16; ++it) {
              const int orow = tok0 + 2 * it + half;
              if (orow >= R || (wg_flag && gload(hot.flags + orow))) continue;  // flagged rows: exact_rows below
              *(TK_GLOBAL v4u *)(gp + it * gstep) = *(const v4u *)(sp + it * 2 * STRIDE);
            }
          }
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      });
    }
  };
  if (hot.out_dtype == TK_BF16) finish(std::integral_constant<int, 2>{});
  else finish(std::integral_constant<int, 4>{});
  if (wg_flag) {  // tokens that hold NaN or Inf: the reference's order, one output at a time
    for (int p = 0; p < PW; ++p) {
      const int ncol = col0 + p * 32 + r32;
      if (ncol >= pr.n) continue;
      for (int rt2 = 0; rt2 < RT2; ++rt2)
        for (int q = 0; q < 4; ++q) {
          const int rowbase = row_base + rt2 * 32 + 8 * q + 4 * kappa;
          const unsigned fl = row_flags(pr, rowbase);
          if (fl) exact_rows(pr, ncol, rowbase, fl);
        }
    }
  }
}

// FORM 0: four waves of 64 rows, the whole column block of 224 outputs, one workgroup per CU (up to 512 registers).
// FORM 1: eight waves of 32 rows, the whole column block, one workgroup per CU (two waves per SIMD).
// FORM 2: four waves of 64 rows over a PART of the column block -- the first half of the grid takes pairs 0..3 (128
//         outputs), the second half pairs 4..6 (96 outputs) -- two workgroups per CU (two waves per SIMD): the one with the
//         narrower part finishes its K loop first and its epilogue runs under the other's matrix instructions.
template <int FORM>
__global__ __launch_bounds__(FORM == 1 ? 512 : 256) __attribute__((amdgpu_waves_per_eu(FORM == 0 ? 1 : 2, FORM == 0 ? 1 : 2))) void
tk_gemm256_kernel(const TkProblem single) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const TkProblem &pr = *single_problem();
  const TkHot hot = make_hot(pr);
  // XCD x = id % 8 owns a sub-grid of sub_m x sub_n blocks and walks it row band by row band: the workgroups an
  // XCD holds at a time share one or two 256-row bands of the operand rows in its L2
  const int sub_m = pr.sub_m, sub_n = pr.sub_n;
  const unsigned blocks = 8u * (unsigned)sub_m * (unsigned)sub_n;
  const unsigned part = FORM == 2 ? (blockIdx.x >= blocks ? 1u : 0u) : 0u;
  const unsigned wg = blockIdx.x - part * blocks;
  const int xcd = (int)(wg & 7u), slot = (int)(wg >> 3);
  const int lm = slot / sub_n, ln = slot - lm * sub_n;
  const int bm = (xcd % pr.xr) * sub_m + lm, bn = (xcd / pr.xr) * sub_n + ln;
  if (lm >= sub_m || bm >= pr.grid_m || bn >= pr.grid_n) return;
  if constexpr (FORM == 0) tk_g256_body<2, TK_G256_PAIRS>(pr, hot, smem, bm, bn * TK_G256_TILES);
  else if constexpr (FORM == 1) tk_g256_body<1, TK_G256_PAIRS>(pr, hot, smem, bm, bn * TK_G256_TILES);
  else if (part == 0) tk_g256_body<2, 4>(pr, hot, smem, bm, bn * TK_G256_TILES);
  else tk_g256_body<2, 3>(pr, hot, smem, bm, bn * TK_G256_TILES + 8);
}

int tk_gemm256_lds_bytes(int form) {
  const int waves = form == 1 ? 8 : 4, pw = form == 2 ? 4 : TK_G256_PAIRS;
  const int stage = waves * TK_G256_WAVE_LDS, loop = 2 * TK_G256_BBUF(pw);
  return stage > loop ? stage : loop;
}

template <int FORM>
static hipError_t launch_gemm256_form(hipStream_t s, const TkProblem *single, unsigned wgs) {
  hipError_t e = tk_raise_lds_limit((const void *)tk_gemm256_kernel<FORM>, tk_gemm256_lds_bytes(FORM));
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(tk_gemm256_kernel<FORM>, dim3(FORM == 2 ? 2 * wgs : wgs), dim3(FORM == 1 ? 512 : 256),
                     (size_t)tk_gemm256_lds_bytes(FORM), s, *single);
  return hipGetLastError();
}

hipError_t tk_launch_gemm256(hipStream_t s, const TkProblem *single, int form) {
  const unsigned wgs = 8u * (unsigned)single->sub_m * (unsigned)single->sub_n;
  if (!wgs) return hipSuccess;
  if (form == 1) return launch_gemm256_form<1>(s, single, wgs);
  if (form == 2) return launch_gemm256_form<2>(s, single, wgs);
  return launch_gemm256_form<0>(s, single, wgs);
}
