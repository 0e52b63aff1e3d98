// Internal declarations shared by the host API and the kernel translation unit.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/tritium_mi355x.h"

// ---- device-private weight layout ("T16") -------------------------------------------------
// A plane is cut into tiles of 16 output rows. Tile t, 256-trit block kb is one contiguous
// 1024-byte chunk at ((t*nb + kb) * 1024). Inside a chunk, lane l = g*16 + r (r = row in tile,
// g = 0..3) owns 16 bytes: bytes [g*16, g*16+16) of the TQ2_0 code block of row t*16+r.
// Byte (g*16 + 4j + b), 2-bit slot s, is trit index
//     kb*256 + (g/2)*128 + s*32 + (g%2)*16 + 4j + b            (crates/tritium-format/src/tq2.rs:15-18)
// Rows past n are filled with 0x55 (all-zero trits). Block scales are dropped.
#define TK_TILE_ROWS 16
#define TK_CHUNK_BYTES 1024
// all-zero chunks kept behind a plane's last chunk (a power of two): a request for a chunk the zero-chunk map marks
// reads copy (chunk index mod this). One copy: spreading the redirected requests over 16 copies (in case they crowded
// a cache channel) measured 2-6% slower on a plane with 75% marked chunks (two planes K=2048 N=8192, 1 / 4 / 16 int8
// tokens: 151 / 148 / 164 -> 155 / 152 / 174 us per 128 layers).
#ifndef TK_ZERO_CHUNKS
#define TK_ZERO_CHUNKS 1
#endif

// More than 64 KiB of dynamic LDS has to be asked for once per kernel AND device (a process may hold a context on
// every GPU of a node): remembered per thread, keyed by both.
static inline hipError_t tk_raise_lds_limit(const void *kernel, int bytes) {
  static thread_local const void *done_kernel[1024];
  static thread_local int done_dev[1024];
  static thread_local int ndone = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  for (int i = 0; i < ndone; ++i)
    if (done_kernel[i] == kernel && done_dev[i] == dev) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return e;
  if (ndone < 1024) {
    done_kernel[ndone] = kernel;
    done_dev[ndone++] = dev;
  }
  return hipSuccess;
}

// ---- base-3 weight stream ("T16B3"), an optional second copy of a plane ----------------------
// The same tiles and K blocks, 832 bytes per chunk instead of 1024: lane l = g*16 + r keeps its 64
// trits (the ones its 16 bytes of the T16 chunk hold) in 13 bytes of five base-3 digits each, encoded
// as TQ1_0 encodes a byte (v = d0*81 + d1*27 + d2*9 + d3*3 + d4 over codes trit+1, byte =
// ceil(v*256/243); digit n decodes as ((uint8)(byte*3^n) * 3) >> 8: crates/tritium-format/src/tq1.rs:18-30,
// crates/tritium-cuda/kernels/tq2_0_add.cu:744-774). Bytes 0..11 of lane l sit at l*12 (three dwords),
// byte 12 at 768 + l. With c[j][s][b] the code of the T16 chunk's dword j, byte b, 2-bit slot s:
//   byte t < 12: digit 0 = c[t/4][3][t%4], digits 1..4 = c[t/3][t%3][0..3]
//   byte 12:     digit 0 = 0,              digits 1..4 = c[3][3][0..3]
// so that digits 1..4 of a byte are one MFMA operand dword (read from a 256-entry table) and digit 0
// of the four bytes of a dword is another (two multiplies by 3 on the even and the odd bytes).
#define TK_B3_CHUNK_BYTES 832
#define TK_B3_TABLE_BYTES 65536  // 256 entries x 64 lanes x 4 bytes: every lane reads its own bank

// ---- activation operand layout ("Ap") -----------------------------------------------------
// int8 rows (R of them), laid out so that one 16-byte read is one MFMA A operand matching the
// B operand obtained from dword j of a weight lane:
//   offset((kb,j,g), row) = (((kb*4 + j)*4 + g) * R + row) * 16,   byte s*4+b inside
// holds q[row][kb*256 + (g/2)*128 + s*32 + (g%2)*16 + 4j + b]  (0 beyond k).

enum { TK_MODE_INT8 = 0, TK_MODE_DIGITS = 1 };

struct TkProblem {
  const uint8_t *codes[TK_MAX_PLANES];
  const uint8_t *codes3[TK_MAX_PLANES];  // the plane's base-3 stream, or null (only the base-3 flow kernel reads it)
  const float *scales[TK_MAX_PLANES];
  const int8_t *ap;          // operand rows, row stride R
  const int32_t *rowsum;     // [R]
  const float *act_scale;    // INT8: [M] or null
  const float *aux;          // INT8 from float: [M] 127/gamma (for the exact fallback)
  const int32_t *exps;       // DIGITS: [M] binary exponent of the fixed-point grid
  const uint32_t *flags;     // [M] non-zero -> row takes the exact sequential fallback (or null)
  const void *raw_act;       // original activations [M,K] for the fallback (or null)
  // kernels that build the operand rows themselves (one launch per call): an RMSNorm in front of the quantization
  // of raw_act (norm_kind 0 = none, 1 = scale w, 2 = scale 1 + w), one token
  const float *norm_w;
  float norm_eps;
  int norm_kind;
  // block-scale planes only: per plane the f32 block scales [(tile, K block), 16 rows], and the sums
  // of every operand row over each K block [nb][R]
  const float *bscale[TK_MAX_PLANES];
  const int32_t *blocksum;
  // Zero-chunk skip (flow kernel): per plane, one bit per 1-KiB chunk (tile * nb + K block), set when all
  // 16 rows of the tile hold only zero trits in that block, or null; a chunk whose bit is set is loaded
  // from the resident all-zero chunk behind the plane's last chunk instead (same bytes, no memory traffic).
  const uint32_t *zmap[TK_MAX_PLANES];
  int zskip;                 // any plane has a map
  void *out;                 // [M,N]
  const void *residual;      // [M,N] in the output's element type, added to every output (one f32 add), or null
  int n, k, nb, R, M;
  int rs;                    // row stride of `ap` in rows (>= R; the GEMM pads it, see tk_api.hip)
  int mode, raw_dtype, out_dtype, planes;
  int tile_begin;            // first launch-wide tile index of this problem
  int n_tiles;               // ceil(n/16)
  int kc;                    // K blocks staged in LDS per pass (decode kernels)
  int group_begin;           // streaming / flow kernels: first workgroup index of this problem
  int run_tiles;             // flow kernel: consecutive tiles per run (S)
  // prefill kernel, K split (single launches with too few workgroups to fill the chip): every output tile
  // is computed by `ksplit` workgroups, each over a slice of the K blocks; their int32 partial sums meet in
  // kpart, and the workgroup that arrives last (kcount) adds them up -- integer adds, so the bits are those
  // of the unsplit kernel -- and runs the epilogue. 0 or 1 = no split.
  int ksplit;
  int32_t *kpart;            // [tile][slice][accumulator register][thread]
  int *kcount;               // [tile], zero between launches
  int grid_m, grid_n;        // GEMM: row blocks and column blocks
  int xr, sub_m, sub_n;      // GEMM: XCDs along M, and the tile sub-grid one XCD owns
};

enum { TK_PREP_A8 = 0, TK_PREP_DIGITS = 1, TK_PREP_I8 = 2 };

// One activation tensor to bring into operand order (one workgroup per token).
struct TkPrep {
  const void *act;      // [m,k] f32 / bf16 (A8, DIGITS) or int8 (I8)
  int8_t *ap;           // operand rows, row stride R (may be null for A8 when only q_rowmajor is wanted)
  int32_t *rowsum;      // [R]
  float *act_scale;     // A8: [m]
  float *aux;           // A8: [m] 127/gamma
  int32_t *exps;        // DIGITS: [m]
  uint32_t *flags;      // [m]
  int8_t *q_rowmajor;   // A8: optional plain [m,k] int8 copy
  size_t k, nb, R;
  size_t rs;            // row stride of `ap` in rows (>= R)
  int act_dtype;
  int row_begin;        // first launch-wide token index of this tensor
  int m;
  // A8 only: RMSNorm of each row in front of the quantization (norm_kind 0 = none, 1 = scale w,
  // 2 = scale 1 + w). A normalized row that holds NaN or Inf is also written to ynorm [m,k] f32,
  // which the exact fallback of such rows reads in place of the raw activation.
  int32_t *blocksum;    // DIGITS, optional: [nb][R] sums of each operand row over one K block
  int norm_kind;
  float norm_eps;
  const float *norm_w;  // [k]
  float *ynorm;
};

struct TkLaunchCfg {
  int planes;   // 1..TK_MAX_PLANES
  int rt;       // row tiles per workgroup (skinny: 1,2,4 ; gemm: 8)
  size_t lds_bytes;
  unsigned grid;
  int waves;    // flow kernel: waves per workgroup (4, or 8 when the operand rows need > 64 KiB of LDS)
  int ring;     // flow kernel: positions in the prefetch ring (2..5)
  int wide_mfma; // flow kernel: 32x32x32 form (17..64 operand rows, row constants in LDS)
  int gemm_nt;  // prefill kernel, one plane: 0 = 64 x 256 outputs per workgroup (4 tiles per wave), 2 = 64 x 128
  int gemm_two_by_two;  // ... the 64 x 128 form with its waves two by two (32 rows x 4 tiles each) instead of side by side
  int tw;       // flow kernel, 16x16x64 form: runs per wave (tk_flow_runs_per_wave)
  int base3;    // flow kernel: stream the planes' base-3 copies (tk_launch_flow3)
  int fused;    // flow kernel, one row tile, one problem: build the operand rows in the kernel (no prep launch)
  int zmap32;   // flow kernel, 32x32x32 form: the instantiations that consult the zero-chunk maps (tk_zskip.hip)
  int swap;     // flow kernel, 16x16x64 form, int8 contract: the second operand order (tk_flow_a8.hip)
};

#ifdef __cplusplus
extern "C++" {
#endif
// kernel launchers (tk_kernels.hip). Return hipError_t from the launch.
hipError_t tk_launch_relayout_tq2(hipStream_t s, const uint8_t *raw, uint8_t *codes, size_t n, size_t nb,
                                  int *invalid_row, float *block_scales);
hipError_t tk_launch_relayout_tq1(hipStream_t s, const uint8_t *raw, uint8_t *codes, size_t n, size_t nb);
// chunk map of a re-laid-out plane: bit c of map set iff chunk c is all 0x55; *count receives the set bits
hipError_t tk_launch_zero_chunk_map(hipStream_t s, const uint8_t *codes, size_t chunks, uint32_t *map, unsigned *count);
// LDS bytes the flow kernel needs for the maps of one workgroup: planes * this many words
size_t tk_flow_zmap_words(size_t tiles_per_wg, size_t nb);
// the 32x32x32 flow kernel's forms that consult the zero-chunk maps (tk_zskip.hip; tk_launch_flow goes there when
// cfg.zmap32 is set): same arguments as tk_launch_flow
hipError_t tk_launch_flow32_zmap(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                                 const TkLaunchCfg &cfg);
// the 16x16x64 flow kernel's forms with weights as the first operand (tk_flow_a8.hip; int8 contract only; tk_launch_flow
// goes there when cfg.swap is set): same arguments as tk_launch_flow
hipError_t tk_launch_flow_swapped(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                                  const TkLaunchCfg &cfg);
hipError_t tk_launch_decode_trits(hipStream_t s, const uint8_t *codes, size_t n, size_t k, size_t nb,
                                  int8_t *trits);
// uniform_m > 0 says that entry j of the table starts at token j * uniform_m (all tensors equally long).
// table_wave_pieces: for a table, the largest piece count (16 * K blocks) of its entries when every entry can
// take the one-wave-per-token kernels (at most 256 pieces, no norm, no per-block sums), else 0.
// table_fast: for a table, 1 (f32) or 2 (bf16) when tk_prep_fast says so for every entry (and the same), else 0.
// table_norm_fast / table_norm_pieces: for a table of quantizations with an RMSNorm in some entry, 1 / 2 when
// tk_prep_norm_fast says so for every entry (and the same), and the largest piece count; else 0.
hipError_t tk_launch_prep(hipStream_t s, int kind, const TkPrep *single, const TkPrep *table, int nprep, int uniform_m,
                          unsigned rows, int table_wave_pieces = 0, int table_fast = 0, int table_norm_fast = 0,
                          int table_norm_pieces = 0);
// 1 / 2: rows of f32 / bf16 that the one-wave-per-token kernels may take without per-element tests (whole K
// blocks, 16-byte aligned, operand rows only); 0 otherwise
int tk_prep_fast(const TkPrep &pp);
int tk_prep_norm_fast(const TkPrep &pp);
void tk_prep_set_team_rows(int rows);  // process-wide: launches of up to `rows` tokens give a token the whole workgroup
hipError_t tk_launch_skinny(hipStream_t s, const TkProblem *single, const TkProblem *table, int nprobs,
                            const TkLaunchCfg &cfg);
// streaming decode kernel: tiles per workgroup for a (planes, rt) pair, and the launcher
int tk_stream_tiles_per_wg(int planes, int rt);
hipError_t tk_launch_stream(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                            const TkLaunchCfg &cfg);
int tk_flow_runs_per_wave(int planes, int rt, int rows);
hipError_t tk_launch_flow(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                          const TkLaunchCfg &cfg);
// base-3 stream (tk_base3.hip): re-encode a T16 plane, and the flow kernel that streams the result.
// The kernel takes 1..3 planes and one or two row tiles (<= 32 operand rows), always with a ring of four
// positions and tk_flow3_runs_per_wave(planes) runs per wave; its LDS holds the decode table
// (TK_B3_TABLE_BYTES) in front of the operand rows.
hipError_t tk_launch_encode_base3(hipStream_t s, const uint8_t *codes, uint8_t *codes3, size_t chunks);
int tk_flow3_runs_per_wave(int planes);
int tk_flow3_waves(int rt);  // waves per workgroup
hipError_t tk_launch_flow3(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                           const TkLaunchCfg &cfg);
int tk_gemm_tiles_per_wg(int planes);
int tk_gemm_lds_bytes(void);
int tk_flow_ring(const int *nbs, const double *weights, int count, int rt, int rows, int tw);
int tk_flow32_runs_per_wave(void);
// block-scale planes (float activations): flow form for <= 64 operand rows resident in LDS, and the
// reference-order kernel for everything else
hipError_t tk_launch_salt_flow(hipStream_t s, const TkProblem *single, const TkLaunchCfg &cfg);
hipError_t tk_launch_salt_seq(hipStream_t s, const TkProblem *single);
hipError_t tk_launch_gemm(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                          const TkLaunchCfg &cfg);
// 128 x 256 prefill kernel (tk_gemm128.hip): one plane, int8 contract, f32 / bf16 rows of whole 16-byte pieces,
// no residual; grid from the problem's XCD split over 128-row x 16-tile blocks
int tk_gemm128_lds_bytes(void);
hipError_t tk_launch_gemm128(hipStream_t s, const TkProblem *single);
// 256 x 224 prefill kernel (tk_gemm256.hip): the same launches as the 128 x 256 kernel; the weight tile is expanded to
// int8 once per workgroup, in LDS. form 0: four waves of 64 rows over the whole column block (224 outputs); 1: eight
// waves of 32 rows; 2: four waves over a part of the column block (128 or 96 outputs), two workgroups per CU. Grid from
// the problem's XCD split over 256-row x 14-tile blocks.
int tk_gemm256_lds_bytes(int form);
hipError_t tk_launch_gemm256(hipStream_t s, const TkProblem *single, int form);
hipError_t tk_launch_seq(hipStream_t s, const TkProblem *single);
// The three gradients of one packed mpGEMM (tk_vjp.hip); a null output is skipped.
hipError_t tk_launch_projected_vjp(hipStream_t s, const uint8_t *codes, size_t nb, size_t n, size_t k, size_t m,
                                   const float *scales, const float *act, const float *grad_output, float *grad_act,
                                   float *grad_w, float *grad_bias);
hipError_t tk_launch_copy(hipStream_t s, void *dst, const void *src, size_t bytes);

// SALT V2 (tk_salt_v2.hip). The resident tensor: codec payload, f16 scales, and per tile the running plane
// index of its first plane (tile_begin[tiles + 1]; the plane count of a tile is the difference).
struct TkSaltV2 {
  const uint8_t *payload;
  const uint16_t *scales;
  const uint32_t *tile_begin;
  unsigned n, k, codec, group;       // group = coefficients per scale: 128 or 64
  unsigned tiles;
  unsigned long long total;          // n * k
};
// tokens one workgroup carries through a weight row, and the LDS a launch needs for rows of k columns
#define TK_SALT_V2_TOKENS 8
size_t tk_salt_v2_lds_bytes(size_t k, size_t group);
// tmp receives the [m,n] results; *flag is raised when an activation or a result is not finite
// terms: workspace of term_tokens * tk_salt_v2_term_floats(t) floats for the lane-per-row form (rows of whole scale
// groups; tk_salt_v2_term_floats is 0 for other matrices), or null: the form that needs none
size_t tk_salt_v2_term_floats(const TkSaltV2 &t);
hipError_t tk_launch_salt_v2_forward(hipStream_t s, const TkSaltV2 &t, const float *act, size_t m, float *tmp, unsigned *flag,
                                     float *terms, size_t term_tokens);
// out[i] = tmp[i] for i < count unless *flag is set (then nothing is written)
hipError_t tk_launch_salt_v2_commit(hipStream_t s, const float *tmp, float *out, size_t count, const unsigned *flag);
hipError_t tk_launch_salt_v2_gather(hipStream_t s, const TkSaltV2 &t, const uint32_t *rows, size_t count, float *out);
#ifdef __cplusplus
}
#endif
