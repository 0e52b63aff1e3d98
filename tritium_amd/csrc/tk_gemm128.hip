// gfx950 prefill GEMM, 128 x 256 outputs per workgroup, one plane, int8 contract.
//
// The 64-row prefill kernels (tk_kernels.hip) are held back by the CU's vector-memory path, not by the
// matrix pipe: every wave loads its own weight chunks into registers and the four waves of a workgroup
// share one 64-row A block, 24-32 KiB of loads per 4-8 MOP. Here eight waves (two row groups of 64 rows x
// four column groups of 64 outputs) share both operands through LDS: per half K block (128 k) a workgroup
// brings in 16 KiB of A rows and 8 KiB of 2-bit weight chunks, all by LDS-DMA (three wave-wide 16-byte
// loads per wave), for 16.8 MOP -- 1.4 KiB per MOP where the 64 x 256 form moves 3.8. A wave computes
// 64 x 64 outputs with v_mfma_i32_32x32x32_i8 (two 32-row A tiles x two pairs of weight tiles: 64
// accumulator registers), reads its A pieces and its 16-byte weight pieces from LDS and expands the 2-bit
// codes exactly as the other kernels do, so the accumulators are the same integers and the outputs carry
// the same bits. (A wave over all 128 rows of 32 outputs -- half the expansion work, 1.7 times the LDS reads --
// measured 4-8% slower.)
//
// LDS: three stages of 24 KiB (A: 8 segments (j, kappa) x 128 rows x 16 B; W: 16 tiles x 512 B = the half
// of each 1-KiB chunk that belongs to this half block), two half blocks in flight, one barrier per half
// block; 1.5 KiB of row constants behind the stages. Two workgroups per CU (four waves per SIMD, at most
// 128 registers). The epilogue stages finished rows through the (then free) stage memory and writes whole
// 16-byte pieces of contiguous row segments, like the 64-row kernels.
//
// Takes: one plane, int8 operand rows (W1.58A8 or int8 input), f32 or bf16 output whose rows are 16-byte
// multiples at a 16-byte aligned address, no residual. Everything else stays with the 64-row kernels.

#include "tk_device.h"

typedef int v16i_g __attribute__((ext_vector_type(16)));

#define TK_G128_THREADS 512
#define TK_G128_HALF_A 16384
#define TK_G128_HALF_W 8192
#define TK_G128_STAGE (TK_G128_HALF_A + TK_G128_HALF_W)
#define TK_G128_STAGES 3
#define TK_G128_CST (TK_G128_STAGES * TK_G128_STAGE)
#define TK_G128_BAND 4

__global__ __launch_bounds__(TK_G128_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void tk_gemm128_kernel(const TkProblem single) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const TkProblem &pr = *single_problem();
  const TkHot hot = make_hot(pr);
  const int tid = (int)threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r16 = lane & 15, h = (lane >> 4) & 1, kappa = lane >> 5;
  const int rg = wave >> 2, cg = wave & 3;  // row group (64 rows), column group (64 outputs)
  const int nb = pr.nb, R = pr.R, n_tiles = pr.n_tiles, rs = pr.rs;
  const uint8_t *codes = pr.codes[0];
  const int8_t *ap = pr.ap;

  // XCD x = id % 8 owns a compact sub-grid of sub_m x sub_n tiles and walks it in bands of TK_G128_BAND
  // row tiles, down the band first (as the 64-row kernels do)
  const unsigned wg = blockIdx.x;
  const int xcd = (int)(wg & 7u), slot = (int)(wg >> 3);
  const int sub_m = pr.sub_m, sub_n = pr.sub_n;
  const int band_sz = TK_G128_BAND * sub_n;
  const int band = slot / band_sz, in_band = slot - band * band_sz;
  const int band_rows = min(TK_G128_BAND, sub_m - band * TK_G128_BAND);
  if (band_rows <= 0) return;
  const int lm = band * TK_G128_BAND + in_band % band_rows, ln = in_band / band_rows;
  const int bm = (xcd % pr.xr) * sub_m + lm, bn = (xcd / pr.xr) * sub_n + ln;
  if (lm >= sub_m || ln >= sub_n || bm >= pr.grid_m || bn >= pr.grid_n) return;
  const int row0 = bm * 128, tile0 = bn * 16;

  // this wave's three DMA instructions of a half block: ids 3*wave .. 3*wave+2 of [A0..A15, W0..W7].
  // A id i: segment i >> 1 (j = seg >> 1, kappa = seg & 1), rows (i & 1) * 64 + lane.
  // W id w: tiles 2w and 2w+1, lane -> tile 2w + (lane >> 5), 16-byte piece lane & 31 of its half chunk.
  const uint8_t *gsrc[3];   // lane address for half block 0 (K block 0, l = 0)
  unsigned kb_step[3];      // bytes from one K block to the next
  unsigned l_step[3];       // bytes from half 0 to half 1 of a K block
  unsigned lds_dst[3];      // wave-uniform offset inside a stage
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int id = wave * 3 + i;
    if (id < 16) {
      const int seg = id >> 1, j = seg >> 1, kap = seg & 1;
      const int row = min(row0 + (id & 1) * 64 + lane, R - 1);
      gsrc[i] = (const uint8_t *)ap + ((size_t)(j * 4 + kap) * (size_t)rs + (size_t)row) * 16;
      kb_step[i] = (unsigned)rs * 256u;  // 16 segments of rs rows of 16 bytes
      l_step[i] = (unsigned)rs * 32u;    // g = 2l + kappa: two segments further
      lds_dst[i] = (unsigned)((seg * 128 + (id & 1) * 64) * 16);
    } else {
      const int w = id - 16;
      const int tile = min(tile0 + 2 * w + (lane >> 5), n_tiles - 1);
      gsrc[i] = codes + (size_t)tile * (size_t)nb * 1024 + (size_t)(lane & 31) * 16;
      kb_step[i] = 1024u;
      l_step[i] = 512u;
      lds_dst[i] = (unsigned)(TK_G128_HALF_A + w * 1024);
    }
  }
  auto issue = [&](int hb, int stage) {
    const unsigned kb = (unsigned)hb >> 1, l = (unsigned)hb & 1u;
#pragma unroll
    for (int i = 0; i < 3; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gsrc[i] + (size_t)kb * kb_step[i] + l * l_step[i]),
                                       (__attribute__((address_space(3))) void *)(smem + (size_t)stage * TK_G128_STAGE + lds_dst[i]),
                                       16, 0, 0);
  };

  // row constants behind the stages: int rowsum[128] | float act_scale[128]
  int *cst_rs = (int *)(smem + TK_G128_CST);
  float *cst_as = (float *)(smem + TK_G128_CST + 512);
  if (tid < 128) {
    const int row = min(row0 + tid, R - 1);
    cst_rs[tid] = gload(hot.rowsum + row);
    cst_as[tid] = hot.act_scale ? gload(hot.act_scale + row) : 1.0f;
  }

  const int HB = 2 * nb;
  issue(0, 0);
  issue(1, 1);  // nb >= 1: a K block has two halves

  v16i_g acc[2][2];
#pragma unroll
  for (int rt2 = 0; rt2 < 2; ++rt2)
#pragma unroll
    for (int y = 0; y < 2; ++y)
#pragma unroll
      for (int c = 0; c < 16; ++c) acc[rt2][y][c] = 0;

  asm volatile("s_waitcnt vmcnt(3)" ::: "memory");  // half block 0 has landed (this wave's part)
  __syncthreads();  // (also publishes the row constants)

  // lane offsets inside a stage: A piece (j, kappa) of row rg*64 + rt2*32 + (lane & 31); weight piece
  // (kappa, r16) of tile cg*4 + 2y + h
  const unsigned a_lane = (unsigned)((kappa * 128 + rg * 64 + (lane & 31)) * 16);
  const unsigned w_lane = (unsigned)(TK_G128_HALF_A + (cg * 4 + h) * 512 + (kappa * 16 + r16) * 16);
  int stage = 0;
  for (int hb = 0; hb < HB; ++hb) {
    const bool more = hb + 2 < HB;
    if (more) issue(hb + 2, stage == 0 ? 2 : stage - 1);  // the stage half block hb-1 just left
    const uint8_t *sb = smem + (size_t)stage * TK_G128_STAGE;
    v4i wp[2];
#pragma unroll
    for (int y = 0; y < 2; ++y) wp[y] = *(const v4i *)(sb + w_lane + y * 1024);
    v4i a_cur[2], a_nxt[2];
#pragma unroll
    for (int rt2 = 0; rt2 < 2; ++rt2) a_cur[rt2] = *(const v4i *)(sb + a_lane + rt2 * 512);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (j < 3) {
#pragma unroll
        for (int rt2 = 0; rt2 < 2; ++rt2) a_nxt[rt2] = *(const v4i *)(sb + a_lane + (j + 1) * 4096 + rt2 * 512);
      }
#pragma unroll
      for (int y = 0; y < 2; ++y) {
        const v4i b = expand_codes((uint32_t)wp[y][j]);
#pragma unroll
        for (int rt2 = 0; rt2 < 2; ++rt2)
          acc[rt2][y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_cur[rt2], b, acc[rt2][y], 0, 0, 0);
      }
      if (j < 3) {
#pragma unroll
        for (int rt2 = 0; rt2 < 2; ++rt2) a_cur[rt2] = a_nxt[rt2];
      }
    }
    // half block hb+1 must have landed; the one issued above may stay in flight.
    // (A bare barrier: __syncthreads() would also drain the loads in flight. Every wave has consumed its
    // LDS reads of this stage in matrix instructions issued above, so the stage may be overwritten. Moving
    // the barrier in front of the last k step, with the next half block's first reads behind it, measured
    // no faster here and 2-4% slower in the 64-row kernels.)
    if (more) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");  // no LDS read of the next half block moves above the barrier
    stage = stage == 2 ? 0 : stage + 1;
  }

  // ---- epilogue: out[m,n] = ((float)(acc - rowsum[m]) * scale[n]) * act_scale[m] ----
  unsigned my_flag = 0;
  if (hot.flags && tid < 128 && row0 + tid < R) my_flag = gload(hot.flags + row0 + tid) ? 1u : 0u;
  const int wg_flag = __syncthreads_or((int)my_flag);
  const bool has_as = hot.act_scale != nullptr;
  float sc[2][1];
  int ncol[2];
#pragma unroll
  for (int y = 0; y < 2; ++y) {
    ncol[y] = (tile0 + cg * 4 + 2 * y + h) * 16 + r16;
    sc[y][0] = ncol[y] < hot.n ? gload(pr.scales[0] + ncol[y]) : 0.0f;
  }
  const int col0 = bn * 256;
  auto finish = [&](auto esz_c) {
    constexpr int ESZ = decltype(esz_c)::value;
    constexpr int HALVES = ESZ == 4 ? 2 : 1, SROWS = 128 / HALVES;  // staging rows per pass
    constexpr int STRIDE = 256 * ESZ + 16, PIECES_ROW = 256 * ESZ / 16, PER16 = 16 / ESZ;
    static_assert(SROWS * STRIDE <= TK_G128_CST, "the staging area is the stage memory");
    uint8_t *lane_base = smem + (size_t)(4 * kappa) * STRIDE + (size_t)((cg * 4 + h) * 16 + r16) * ESZ;
#pragma unroll
    for (int hh = 0; hh < HALVES; ++hh) {
      if (hh > 0) __syncthreads();
#pragma unroll
      for (int rt2 = 0; rt2 < 2; ++rt2) {
        if (HALVES == 2 && rt2 != hh) continue;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rl = rg * 64 + rt2 * 32 + 8 * q + 4 * kappa;             // first of this lane's 4 rows, tile-local
          const int sl = (HALVES == 2 ? rg * 32 : rg * 64 + rt2 * 32) + 8 * q;  // staging row less 4 * kappa
          RowConst rc;
          const v4i rs4 = *(const v4i *)(cst_rs + rl);
          const float4 as4 = *(const float4 *)(cst_as + rl);
          rc.rs[0] = rs4.x; rc.rs[1] = rs4.y; rc.rs[2] = rs4.z; rc.rs[3] = rs4.w;
          rc.as[0] = as4.x; rc.as[1] = as4.y; rc.as[2] = as4.z; rc.as[3] = as4.w;
#pragma unroll
          for (int y = 0; y < 2; ++y) {
            const v4i av[1] = {v4i{acc[rt2][y][4 * q], acc[rt2][y][4 * q + 1], acc[rt2][y][4 * q + 2], acc[rt2][y][4 * q + 3]}};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float f = int8_value<1>(av, r, sc[y], rc, has_as);
              uint8_t *dst = lane_base + (size_t)(sl + r) * STRIDE + y * 32 * ESZ;
              if (ESZ == 2) *(uint16_t *)dst = f32_to_bf16_hw(f); else *(float *)dst = f;
            }
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int it = 0; it < SROWS * PIECES_ROW / TK_G128_THREADS; ++it) {
        const int pc = it * TK_G128_THREADS + tid;
        const int srow = pc / PIECES_ROW, piece = pc % PIECES_ROW;
        const int orow = row0 + (HALVES == 2 ? (srow >> 5) * 64 + hh * 32 + (srow & 31) : srow);
        const int c = col0 + piece * PER16;
        if (orow >= R || c >= hot.n) continue;
        if (wg_flag && gload(hot.flags + orow)) continue;  // written by exact_rows below
        *(TK_GLOBAL v4u *)((uint8_t *)hot.out + ((size_t)orow * hot.n + c) * ESZ) = *(const v4u *)(smem + (size_t)srow * STRIDE + piece * 16);
      }
    }
  };
  if (hot.out_dtype == TK_BF16) finish(std::integral_constant<int, 2>{});
  else finish(std::integral_constant<int, 4>{});
  if (wg_flag) {
    for (int y = 0; y < 2; ++y) {
      if (ncol[y] >= pr.n) continue;
      for (int rt2 = 0; rt2 < 2; ++rt2)
        for (int q = 0; q < 4; ++q) {
          const int rowbase = row0 + rg * 64 + rt2 * 32 + 8 * q + 4 * kappa;
          const unsigned fl = row_flags(pr, rowbase);
          if (fl) exact_rows(pr, ncol[y], rowbase, fl);
        }
    }
  }
}

int tk_gemm128_lds_bytes(void) { return TK_G128_CST + 1536; }

hipError_t tk_launch_gemm128(hipStream_t s, const TkProblem *single) {
  const unsigned wgs = 8u * (unsigned)single->sub_m * (unsigned)single->sub_n;
  if (!wgs) return hipSuccess;
  hipError_t e = tk_raise_lds_limit((const void *)tk_gemm128_kernel, 128 * 1024);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(tk_gemm128_kernel, dim3(wgs), dim3(TK_G128_THREADS), (size_t)tk_gemm128_lds_bytes(), s, *single);
  return hipGetLastError();
}
