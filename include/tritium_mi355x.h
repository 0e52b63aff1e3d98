/*
 * tritium_mi355x.h — C ABI of the MI355X (gfx950) packed-ternary linear-layer kernel library.
 *
 * This is the boundary a Tritium backend crate binds over FFI: plain pointers and sizes, integer
 * status codes, no C++ or framework types. Each entry point names the reference interface it
 * stands behind (paths are relative to the reference checkout).
 *
 * Conventions (borrowed from the reference's own C ABI, crates/tritium-ffi/src/lib.rs:9-28,
 * crates/tritium-ffi/include/tritium.h:19-43):
 *   - every call returns a tk_status; 0 is success;
 *   - the message for the last failure on the calling thread is tk_last_error();
 *   - null pointers are checked and reported as TK_ERR_INVALID_INPUT, never dereferenced;
 *   - nothing here panics or aborts on bad input (crates/tritium-spec/src/lib.rs:380-381).
 *
 * Shapes follow GemmShape (crates/tritium-core/src/shape.rs:10-38): C[M,N] = A[M,K] · Wᵀ with W
 * the [N,K] ternary weight, row-major, output-major. All matrices are row-major.
 */
#ifndef TRITIUM_MI355X_H
#define TRITIUM_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One code per BackendError variant (crates/tritium-spec/src/lib.rs:382-405). */
typedef enum tk_status {
  TK_OK = 0,
  TK_ERR_SHAPE_MISMATCH = 1,     /* BackendError::ShapeMismatch{expected,got}: see tk_last_mismatch */
  TK_ERR_UNSUPPORTED_FORMAT = 2, /* BackendError::UnsupportedFormat */
  TK_ERR_OUT_OF_MEMORY = 3,      /* BackendError::OutOfMemory{requested}: see tk_last_mismatch */
  TK_ERR_INVALID_INPUT = 4,      /* BackendError::InvalidInput */
  TK_ERR_BACKEND = 5             /* BackendError::Backend (any device error, stringified) */
} tk_status;

/* TernaryFormat (crates/tritium-core/src/dtype.rs:89-107). I2sInt8 is answered with
 * TK_ERR_UNSUPPORTED_FORMAT, as the CPU backend does (crates/tritium-cpu/src/lib.rs:153-159). */
typedef enum tk_format { TK_FORMAT_TQ1_0 = 1, TK_FORMAT_TQ2_0 = 2, TK_FORMAT_I2S_INT8 = 3 } tk_format;

/* Element types of device-resident activations and outputs. */
typedef enum tk_dtype { TK_F32 = 0, TK_BF16 = 1, TK_I8 = 2, TK_I32 = 3 } tk_dtype;

#define TK_MAX_PLANES 4

typedef struct tk_ctx tk_ctx;         /* one device + one stream; Send + Sync, calls serialised inside */
typedef struct tk_weights tk_weights; /* a DeviceBuffer (crates/tritium-spec/src/lib.rs:147-158) */

/* DeviceCaps (crates/tritium-spec/src/caps.rs:7-20) plus what the roofline report needs. */
typedef struct tk_device_info {
  char name[128];
  char arch[32];
  uint64_t total_memory_bytes;
  int compute_units;
  int clock_khz;
  int memory_clock_khz;
  int memory_bus_bits;
  int wavefront_size;
  int lds_bytes_per_cu;
} tk_device_info;

/* ---- lifetime: BackendEntry::init (crates/tritium-runtime/src/lib.rs:73-110) and
 *      RocmBackend::new(ordinal) (crates/tritium-rocm/src/rocm.rs:234-300) ---- */
int tk_init(int device, tk_ctx **out);
/* Frees the context's workspaces. Weight buffers and groups created on it stay valid to FREE (not to
 * use) afterwards, in any order: the stream lives until the last of them is gone. */
void tk_destroy(tk_ctx *ctx);
const char *tk_last_error(void);
/* expected/got of the last ShapeMismatch, or requested/0 of the last OutOfMemory, on this thread */
void tk_last_mismatch(size_t *expected, size_t *got);
/* TernaryBackend::device_id / capabilities (crates/tritium-spec/src/lib.rs:166-186) */
const char *tk_device_id(const tk_ctx *ctx); /* "mi355x:<ordinal>" */
int tk_device_info_get(const tk_ctx *ctx, tk_device_info *out);
int tk_device_count(int *count);

/* ---- host-side packing: tritium-format row packers as TernaryLinear::pack_rows uses them
 *      (crates/tritium-format/src/rows.rs:61-151, tq2.rs:21-81, tq1.rs:36-121,
 *       crates/tritium-nn/src/layers/linear.rs:143-185). Block scale is f16 1.0. ---- */
size_t tk_packed_len(size_t n, size_t k, int format); /* 0 for an unsupported format */
int tk_pack_rows(const int8_t *trits, size_t trits_len, size_t n, size_t k, int format,
                 uint8_t *out, size_t out_len);
int tk_unpack_rows(const uint8_t *packed, size_t packed_len, size_t n, size_t k, int format,
                   int8_t *trits, size_t trits_len);

/* ---- zero-block bitmaps of packed TQ2_0 rows: compute_zero_bitmaps
 *      (crates/tritium-format/src/tq2.rs:101-181). words [n * ceil(nb/32)], nb = ceil(k/256): bit b%32 of
 *      word r*ceil(nb/32) + b/32 is set when block b of row r holds only zero trits (64 code bytes 0x55;
 *      the scale bytes do not count). Rows are row_bytes apart. Short rows or buffers ->
 *      TK_ERR_INVALID_INPUT; k == 0 -> TK_OK, nothing written. This is the per-row map the reference's
 *      sparse decode kernels take; the device keeps its own map at the granularity it streams
 *      (tk_set_zero_skip). ---- */
int tk_compute_zero_bitmaps(const uint8_t *packed, size_t packed_len, size_t n, size_t k, size_t row_bytes,
                            uint32_t *words, size_t words_len);

/* ---- I2_S ingest: convert_i2s_to_tq2_0 (crates/tritium-format/src/i2s_int8.rs:36-68) over
 *      unpack_i2s_tensor (crates/tritium-format/src/i2s.rs:70-158). payload = n*k/4 quant bytes
 *      (32-byte blocks of 128 elements of the flat [n,k] tensor, code = trit + 1, code 3 rejected)
 *      + one little-endian f32 per-tensor scale (longer payloads, e.g. GGUF padding, are fine).
 *      out receives n rows of TQ2_0 blocks with unit block scales, *scale the tensor's scale, which
 *      the caller broadcasts as the per-channel scale. n*k must be a multiple of 128. ---- */
size_t tk_i2s_payload_len(size_t n, size_t k); /* n*k/4 + 4; 0 when n*k is not a multiple of 128 */
int tk_convert_i2s_to_tq2_0(const uint8_t *payload, size_t payload_len, size_t n, size_t k,
                            uint8_t *out, size_t out_len, float *scale);

/* ---- GGUF container (v2/v3): read_gguf and its accessors (crates/tritium-format/src/gguf.rs:
 *      183-292, 360-400, 460-664). Parses header, metadata table and tensor table of a file held in
 *      memory; payloads stay in the caller's buffer, which is not retained. Total: no input reads
 *      out of bounds. A failed parse returns TK_ERR_INVALID_INPUT and reports the GgufError variant
 *      (and the value UnsupportedVersion / InvalidBoolean / UnknownValueType carry). ---- */
typedef struct tk_gguf tk_gguf;
typedef enum tk_gguf_error { /* GgufError (crates/tritium-format/src/gguf.rs:63-96), in its order */
  TK_GGUF_OK = 0,
  TK_GGUF_BAD_MAGIC = 1,
  TK_GGUF_UNSUPPORTED_VERSION = 2,
  TK_GGUF_TRUNCATED = 3,
  TK_GGUF_STRING_TOO_LONG = 4,
  TK_GGUF_DIMS_OVERFLOW = 5,
  TK_GGUF_INVALID_TENSOR_SHAPE = 6,
  TK_GGUF_INVALID_ALIGNMENT = 7,
  TK_GGUF_INVALID_BOOLEAN = 8,
  TK_GGUF_OFFSET_OUT_OF_BOUNDS = 9,
  TK_GGUF_UNKNOWN_VALUE_TYPE = 10,
  TK_GGUF_INVALID_UTF8 = 11
} tk_gguf_error;
/* TensorInfo (gguf.rs:360-374). dims are fastest-varying first; offset is relative to
 * tk_gguf_tensor_data_offset; n_bytes is 0 for a type the reader does not size (I2_S among them).
 * name points into the tk_gguf and lives as long as it. */
typedef struct tk_gguf_tensor {
  const char *name;
  uint32_t n_dims;
  uint64_t dims[8];
  uint32_t ggml_type;
  uint64_t offset;
  uint64_t n_bytes;
} tk_gguf_tensor;
int tk_gguf_open(const uint8_t *buf, size_t len, tk_gguf **out, int *error_kind, uint64_t *error_detail);
void tk_gguf_close(tk_gguf *g);
uint32_t tk_gguf_version(const tk_gguf *g);
uint64_t tk_gguf_alignment(const tk_gguf *g); /* general.alignment, 32 when absent */
uint64_t tk_gguf_tensor_data_offset(const tk_gguf *g);
size_t tk_gguf_tensor_count(const tk_gguf *g);
size_t tk_gguf_metadata_count(const tk_gguf *g);
/* The getters below answer like Option: 1 = Some (and *out written), 0 = None. */
int tk_gguf_tensor_at(const tk_gguf *g, size_t index, tk_gguf_tensor *out);
int tk_gguf_tensor_find(const tk_gguf *g, const char *name, tk_gguf_tensor *out); /* GgufFile::tensor: first match */
/* GgufFile::get_metadata(key) followed by GgufValue::as_* with the reference's coercions. index < 0
 * addresses the key's value, index >= 0 element `index` of its array value. value_type is the GGUF
 * metadata type id (0..12; 9 = array, for which child_type and array_len are filled). */
int tk_gguf_meta_type(const tk_gguf *g, const char *key, long long index, uint32_t *value_type,
                      uint32_t *child_type, uint64_t *array_len);
int tk_gguf_meta_u64(const tk_gguf *g, const char *key, long long index, uint64_t *out);
int tk_gguf_meta_i64(const tk_gguf *g, const char *key, long long index, int64_t *out);
int tk_gguf_meta_f64(const tk_gguf *g, const char *key, long long index, double *out);
int tk_gguf_meta_f32(const tk_gguf *g, const char *key, long long index, float *out);
int tk_gguf_meta_bool(const tk_gguf *g, const char *key, long long index, int *out);
int tk_gguf_meta_str(const tk_gguf *g, const char *key, long long index, const char **out, size_t *len);
/* TensorInfo::element_count (gguf.rs:392-398); overflow -> TK_ERR_INVALID_INPUT */
int tk_gguf_element_count(const tk_gguf_tensor *t, uint64_t *out);
/* Where a tensor's payload lies in the file: the model loader's payload()
 * (crates/tritium-nn/src/model/weights.rs:146-166), which sizes I2_S as elements/4 + 32. */
int tk_gguf_tensor_payload(const tk_gguf *g, size_t file_len, const tk_gguf_tensor *t,
                           uint64_t *abs_offset, uint64_t *len);
/* ---- ternary tensor -> packed rows + one scale per output row: load_ternary
 *      (crates/tritium-nn/src/model/weights.rs:177-333). dims must be [k, n]; type I2_S (36), TQ1_0
 *      (34) or TQ2_0 (35), anything else -> TK_ERR_UNSUPPORTED_FORMAT. I2_S comes out as TQ2_0 rows
 *      with the tensor's f32 scale on every row. TQ rows are copied in their own format; a block
 *      whose f16 scale is 0 gets zero trits; block scales must agree within a row (else
 *      TK_ERR_BACKEND); rows that differ keep their own scales, all-zero rows then take the first
 *      nonzero one; with one scale for the whole tensor the f32 metadata value
 *      "tritium.i2s_scale.<name>" replaces it when present (it must round to the same f16).
 *      packed_len = tk_packed_len(n, k, format) and row_scales_len = n from tk_gguf_ternary_shape. */
int tk_gguf_ternary_shape(const tk_gguf *g, const char *name, size_t *n, size_t *k, int *format);
int tk_gguf_load_ternary(const tk_gguf *g, const uint8_t *file, size_t file_len, const char *name,
                         uint8_t *packed, size_t packed_len, float *row_scales, size_t row_scales_len);

/* ---- TernaryBackend::upload_weights (crates/tritium-spec/src/lib.rs:188-200;
 *      crates/tritium-cpu/src/lib.rs:262-300; crates/tritium-rocm/src/rocm.rs:446-475).
 * Copies; the returned handle owns device memory until tk_free_weights. `packed` is the byte
 * stream tritium-format writes: n rows of ceil(k/256) blocks of 66 (TQ2_0) or 54 (TQ1_0) bytes.
 * Wrong length -> TK_ERR_INVALID_INPUT. The bytes are re-laid out once into a device-private
 * 16-row tile order; block scales are not kept (the path ignores them,
 * crates/tritium-cpu/src/lib.rs:19-21,202-205). ---- */
int tk_upload_weights(tk_ctx *ctx, const uint8_t *packed, size_t packed_len, size_t n, size_t k,
                      int format, tk_weights **out);
/* tk_convert_i2s_to_tq2_0 followed by tk_upload_weights of the result (format TQ2_0): what a loader
 * of a BitNet I2_S checkpoint calls per weight tensor. */
int tk_upload_weights_i2s(tk_ctx *ctx, const uint8_t *payload, size_t payload_len, size_t n, size_t k,
                          tk_weights **out, float *scale);
/* tk_gguf_load_ternary followed by tk_upload_weights: one weight tensor of a GGUF checkpoint onto
 * the device; row_scales [n] is what the caller passes as the per-channel scales of mpgemm. */
int tk_upload_weights_gguf(tk_ctx *ctx, const tk_gguf *g, const uint8_t *file, size_t file_len,
                           const char *name, tk_weights **out, float *row_scales, size_t row_scales_len);
void tk_free_weights(tk_weights *w);
size_t tk_weights_len_bytes(const tk_weights *w); /* DeviceBuffer::len_bytes: the uploaded length */
size_t tk_weights_n(const tk_weights *w);
size_t tk_weights_k(const tk_weights *w);
int tk_weights_format(const tk_weights *w);
/* Zero-chunk skip: what the reference's sparse decode kernels do with per-row bitmaps
 * (crates/tritium-cuda/kernels/tq2_0_add.cu:330-401,504-571), at the granularity this layout streams.
 * At upload every 1-KiB chunk (16 rows x 256 trits) that holds only zero trits is marked; when at least
 * 0.5% of a plane's chunks are (the reference's BITMAP_MIN_ZERO_BLOCK_FRAC,
 * crates/tritium-cuda/src/cuda/mod.rs:384-405) the map is kept, and the bandwidth-bound decode kernel
 * then fetches such chunks from one resident all-zero chunk instead of from memory: same bytes, same
 * arithmetic, identical bits, less traffic. Planes without such structure (i.i.d. trits have none)
 * carry no map and take the plain path. tk_set_zero_skip acts on later uploads: 0 = by the threshold,
 * 1 = never keep a map, 2 = always. tk_weights_zero_chunks reports what an upload found. */
int tk_set_zero_skip(tk_ctx *ctx, int mode);
/* Operand order of the matrix instruction in the decode kernel (both of its forms) under the int8 contract: 1 (default) =
 * weights first, so that a lane finishes four consecutive output channels of one token and writes them with one store;
 * 0 = activations first (four tokens of one channel per lane, four narrow stores), the order the float contract keeps.
 * Same integers, same epilogue arithmetic, identical bits; a tuning and test knob without a counterpart in the
 * reference. */
int tk_set_flow_operand_order(tk_ctx *ctx, int weights_first);
/* Waves per workgroup of the decode kernel where a CU has LDS room for the operand rows of one workgroup only (17..32
 * rows that take more than 80 KiB): 0 = automatic, 8 = eight (two per SIMD), 16 = sixteen (four per SIMD) wherever a
 * form of 1024 threads exists (16x16x64 form, one or two planes: every launch under the int8 contract with weights
 * first, grouped launches otherwise). Automatic: sixteen for one plane when the launch has tiles for every CU. Same
 * bits; a tuning and test knob without a counterpart in the reference. */
int tk_set_flow_workgroup_waves(tk_ctx *ctx, int waves);
int tk_weights_zero_chunks(const tk_weights *w, size_t *zero, size_t *total, int *map_kept);
/* Base-3 weight stream: the decode GEMV of the reference that reads TQ1_0's five-trits-per-byte codes and
 * unpacks them in the kernel (crates/tritium-cuda/kernels/tq2_0_add.cu:744-774,796-913). Here: a second
 * device copy of a plane in which every byte is a TQ1_0-coded group of five trits (52 bytes per 256
 * trits where the 2-bit layout holds 64), regrouped for the int8 matrix instruction, kept BESIDE the 2-bit
 * codes (memory: +81%). Decode launches whose operand rows stay in LDS (at most 32 rows: up to 32 int8
 * tokens or 8 float tokens; at most three planes) then stream the base-3 copy and decode it in the
 * kernel; every other launch reads the 2-bit codes. Same integers, identical bits.
 * tk_set_base3_stream acts on later uploads: 0 = no base-3 copy (default), 1 = uploads in TQ1_0 keep
 * one, 2 = every upload does. tk_weights_base3_bytes: size of a buffer's base-3 copy, 0 if it has none. */
int tk_set_base3_stream(tk_ctx *ctx, int mode);
size_t tk_weights_base3_bytes(const tk_weights *w);
/* Debug/parity aid: decode the device-resident planes back to [n,k] trits. */
int tk_weights_download_trits(tk_ctx *ctx, const tk_weights *w, int8_t *trits, size_t trits_len);

/* ---- TernaryBackend::mpgemm (crates/tritium-spec/src/lib.rs:202-215; oracle:
 *      crates/tritium-cpu/src/lib.rs:302-345). Host slices in, host slice out, synchronous.
 *      out[m,n] = scales[n] · Σ_k act[m,k] · trit[n,k]; `out` fully overwritten.
 * Errors: act/scales/out length -> TK_ERR_SHAPE_MISMATCH; weights n/k/format differ from the
 * call's -> TK_ERR_INVALID_INPUT (the CPU backend's choice, crates/tritium-cpu/src/lib.rs:123-135);
 * a TQ2_0 plane holding the reserved code -> TK_ERR_BACKEND. m == 0 or n == 0 -> TK_OK, no launch. */
int tk_mpgemm(tk_ctx *ctx, const float *act, size_t act_len, const tk_weights *weights,
              const float *scales, size_t scales_len, size_t m, size_t n, size_t k, int format,
              float *out, size_t out_len);

/* ---- TernaryBackend::mpgemm_with_act_quant (crates/tritium-spec/src/lib.rs:228-318) and the
 *      whole of TernaryLinear::forward (crates/tritium-nn/src/layers/linear.rs:229-280):
 *      per-token int8 absmax quant on the device, exact int32 contraction, then
 *      out[m,n] = ((float)acc · scales[n]) · act_scale[m]. Never refuses. ---- */
int tk_mpgemm_with_act_quant(tk_ctx *ctx, const float *act, size_t act_len,
                             const tk_weights *weights, const float *scales, size_t scales_len,
                             size_t m, size_t n, size_t k, int format, float *out, size_t out_len);

/* ---- TernaryBackend::mpgemm_projected_vjp (crates/tritium-spec/src/lib.rs:93-117 the operands,
 *      :217-232 the method; oracle: crates/tritium-cpu/src/lib.rs:347-395 ->
 *      crates/tritium-cpu/src/kernel.rs:199-317; device precedent
 *      crates/tritium-cuda/src/cuda/backend.rs:8683-8760). Host slices in and out, synchronous.
 *        grad_act[m,k] = sum_n grad_output[m,n] * (trit[n,k] * scales[n])
 *        grad_w[n,k]   = sum_m grad_output[m,n] * act[m,k]     (w.r.t. P[n,k] = scales[n]*trit[n,k])
 *        grad_bias[n]  = sum_m grad_output[m,n]                (grad_bias == NULL: Option::None)
 *      every sum in index order with unfused f32 operations, i.e. the bits of the CPU backend's
 *      scalar path (the reference's own bar between backends is 1e-4 relative,
 *      crates/tritium-cuda/src/cuda/tests.rs:733). All outputs are fully overwritten on success and
 *      untouched on error. TQ2_0 and TQ1_0 buffers are both taken, as by the CPU backend.
 * Errors, in the CPU backend's order: buffer n/k/format differ from the call's -> TK_ERR_INVALID_INPUT;
 * a plane holding the reserved code -> TK_ERR_BACKEND ("unpack row R: decoded value 2 outside ternary
 * range"); act, scales, grad_output, grad_act, grad_w, grad_bias length -> TK_ERR_SHAPE_MISMATCH.
 * m == 0 or n == 0: outputs zero-filled; k == 0: grad_bias still summed. */
int tk_mpgemm_projected_vjp(tk_ctx *ctx, const float *act, size_t act_len, const tk_weights *weights,
                            const float *scales, size_t scales_len, const float *grad_output,
                            size_t grad_output_len, size_t m, size_t n, size_t k, int format,
                            float *grad_act, size_t grad_act_len, float *grad_w, size_t grad_w_len,
                            float *grad_bias, size_t grad_bias_len);

/* ---- device-resident extension, reached through TernaryBackend::as_concrete
 *      (crates/tritium-spec/src/lib.rs:320-332); precedent: the CUDA backend's device-resident
 *      decode (crates/tritium-cuda/src/cuda/mod.rs:1029-1064,2998-3041). All pointers below are
 *      device pointers on ctx's device; calls enqueue on ctx's stream and do not synchronise. ---- */

/* One additive-plane linear layer: `planes` weight handles with identical n,k and one per-channel
 * scale vector (device, [n] f32) per plane. */
typedef struct tk_linear_desc {
  const tk_weights *planes[TK_MAX_PLANES];
  const float *scales[TK_MAX_PLANES];
  int n_planes;
} tk_linear_desc;

/* quantize_act_int8 on the device (crates/tritium-spec/src/lib.rs:351-378;
 * precedent crates/tritium-cuda/kernels/tq2_0_imma.cu:84-141): act [m,k] f32 or bf16 ->
 * q [m,k] int8 row-major and act_scale [m] f32. Rows holding NaN or Inf cannot be represented in
 * int8; *their* q is zero and the row is reported in nonfinite_rows (may be null). */
int tk_act_quant_i8(tk_ctx *ctx, const void *act, int act_dtype, size_t m, size_t k, int8_t *q,
                    float *act_scale, uint32_t *nonfinite_rows);

/* Float-activation linear (BASELINE configs 1 and 2): act [m,k] f32 or bf16,
 * out[m,n] = Σ_p scales_p[n] · Σ_k act[m,k]·trit_p[n,k], out f32 or bf16.
 * Accuracy. A token is contracted exactly on a 31-bit fixed-point grid of spacing 2^(E-30),
 * 2^(E-1) <= max|act[m,:]| < 2^E. With D the exact dot product of an output of one plane,
 *     |value - D| <= n_poor · 2^(E-31) + 1.5 ulp(value),
 * n_poor = the non-zero elements under the output's non-zero trits that neither lie on the grid
 * exactly (as int8-valued activations and most of a bf16 token do) nor reach 2^(E-15) in magnitude.
 * The reference's k-ordered f32 fold (crates/tritium-core/src/reference.rs:42-51) is itself only within
 * ~sqrt(K)·2^-24·|partial sums| of D; on ordinary tokens the two agree to ~1e-6 of the largest output.
 * A zero trit makes the fold skip an activation, so an output can miss a token's largest elements and be
 * small next to its maximum. Tokens where that would show -- the rounding noise n_poor·2^(2E-62)/3 of the
 * token exceeds 2^-30 of the energy left without its 96 largest elements, e.g. one activation 2^15 or more
 * times the rest -- and tokens holding NaN or Inf are computed in the reference's own order instead
 * (bit-identical to the CPU backend, and slow: one sequential walk over K per output). */
int tk_linear_float(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype,
                    size_t m, void *out, int out_dtype);

/* W1.58A8 linear on float activations: quantize per token, contract in int32, fold
 * out[m,n] = (Σ_p (float)acc_p · scales_p[n]) · act_scale[m]. Chooses the decode GEMV or the
 * prefill MFMA GEMM by m (crossover: tk_set_gemm_min_m). */
int tk_linear_a8(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype,
                 size_t m, void *out, int out_dtype);

/* tk_linear_a8 for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc, code that must not allocate while another thread captures a HIP graph). No counterpart in the
 * reference. Same arguments and same bits as tk_linear_a8 (the same kernels, except that a narrow prefill
 * launch which tk_linear_a8 would split over K runs unsplit here: the split needs a workspace that grows with
 * the launch); the workspace of the call (operand rows, row sums, per-token scales and flags) lives in a
 * static device array of TK_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process
 * ends, and the call makes no hipMalloc, hipFree or other allocating call. The launches go to the context's
 * own stream, as those of every other entry point do. The workspace takes about (m + 16) * ceil(k/256) * 256
 * bytes: 64 tokens at k = 17408 (1.4 MB) and 2048 tokens at k = 3584 (7.4 MB) are about the largest shapes
 * that fit; one that does not (e.g. 2048 tokens at k = 8192, 16.9 MB) is answered with TK_ERR_INVALID_INPUT.
 * Every call on one GPU shares that GPU's array: calls that overlap on one GPU (two contexts of a device, two
 * threads) race and must be serialised by the caller. */
#define TK_NOALLOC_SCRATCH_BYTES ((size_t)8 << 20)
int tk_linear_a8_noalloc(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype,
                         size_t m, void *out, int out_dtype);

/* RMSNorm in front of the per-token int8 quantization, as one launch: what the CUDA decode calls
 * launch_rmsnorm_quant before the q/k/v and gate/up projections
 * (crates/tritium-cuda/src/cuda/mod.rs:1029-1040). y[i] = (x[i] * inv) * s(w[i]),
 * inv = 1 / sqrt(sum_squares / k + eps), s(w) = w or, zero_centered != 0, 1 + w
 * (crates/tritium-nn/src/ops/rmsnorm.rs:43-96); the sum of squares folds in the reference's
 * canonical order (256 slots, then a power-of-two tree, rmsnorm.rs:21-35), so the result has the
 * bits of the host's rmsnorm followed by quantize_act_int8
 * (crates/tritium-cuda/src/cuda/tests.rs:4675-4771). weight is a device pointer to k floats. */
typedef struct tk_rmsnorm {
  const float *weight;
  float eps;
  int zero_centered;
} tk_rmsnorm;
/* x [m,k] f32 or bf16 -> q [m,k] int8 row-major and act_scale [m]; rows whose normalized values
 * hold NaN or Inf are reported as in tk_act_quant_i8. */
int tk_rmsnorm_quant_i8(tk_ctx *ctx, const void *x, int x_dtype, const tk_rmsnorm *norm, size_t m, size_t k,
                        int8_t *q, float *act_scale, uint32_t *nonfinite_rows);
/* tk_linear_a8 on RMSNorm(x): norm, quantization and operand staging in one launch, then the
 * contraction. */
int tk_linear_rmsnorm_a8(tk_ctx *ctx, const tk_linear_desc *layer, const void *x, int x_dtype,
                         const tk_rmsnorm *norm, size_t m, void *out, int out_dtype);

/* Same contraction on activations that are already int8 (q [m,k]) with their per-token scales
 * (act_scale [m], may be null for 1.0): what the CUDA decode calls gemm_prequantized
 * (crates/tritium-cuda/src/cuda/mod.rs:1029-1064). out_dtype TK_I32 (one plane only) stores the
 * raw int32 accumulators Σ_k q·trit instead of the scaled output. */
int tk_linear_i8(tk_ctx *ctx, const tk_linear_desc *layer, const int8_t *q, const float *act_scale,
                 size_t m, void *out, int out_dtype);

/* The same two calls with a fused residual add, out[m,n] = residual[m,n] + value (one f32 add after the
 * scale multiplies): the epilogue of tq2_0_add_mpgemm_tiled_i8_scaled_residual and its TQ1_0 twin
 * (crates/tritium-cuda/kernels/tq2_0_add.cu:577-637,856-913), which saves the decode step a separate
 * residual_add launch and memory pass after the o and down projections. residual is a device pointer to
 * [m,n] elements of the output's type (f32 or bf16; bf16 is widened, added in f32, rounded once) and may
 * be the output itself. */
int tk_linear_a8_residual(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype,
                          size_t m, const void *residual, void *out, int out_dtype);
int tk_linear_i8_residual(tk_ctx *ctx, const tk_linear_desc *layer, const int8_t *q, const float *act_scale,
                          size_t m, const void *residual, void *out, int out_dtype);

/* ---- block-scale additive planes (SALT): every plane is a TQ2_0 tensor whose per-256-block f16
 *      scales count, W[n,k] = Σ_p s_p[n, k/256] · trit_p[n,k] (crates/tritium-format/src/salt.rs:1-19),
 *      out[m,n] = Σ_k act[m,k] · W[n,k] on float activations. The host definition dequantizes the
 *      row (planes in order) and folds one f32 accumulator over k
 *      (salt.rs:720-738, crates/tritium-nn/src/layers/packed_salt.rs:585-628); the reference's GPU
 *      kernel takes the planes plane-major and is held to 1e-4 of that
 *      (crates/tritium-cuda/kernels/tq2_0_add.cu:640-719). ---- */
/* tk_upload_weights of TQ2_0 rows that also keeps the block scales (device f32, 64 B per KiB of codes) */
int tk_upload_weights_scaled(tk_ctx *ctx, const uint8_t *packed, size_t packed_len, size_t n, size_t k,
                             tk_weights **out);
typedef struct tk_salt_desc {
  const tk_weights *planes[TK_MAX_PLANES]; /* each from tk_upload_weights_scaled, same [n,k] */
  int n_planes;
} tk_salt_desc;
/* act [m,k] f32 or bf16, out [m,n] f32 or bf16. Tokens run on the matrix cores, block by block,
 * 16 at a time (within 1e-4 of the host definition, normally ~1e-6; more than 16 tokens stream the
 * planes once per 16); rows too long for LDS (K beyond ~9,800) and tokens holding NaN or Inf take
 * the host's order exactly (slow). A block scale that is itself infinite or NaN makes its outputs
 * non-finite here and NaN on the host (which multiplies it with the zero trits too). */
int tk_linear_salt(tk_ctx *ctx, const tk_salt_desc *layer, const void *act, int act_dtype, size_t m,
                   void *out, int out_dtype);
/* The host's order for every output: bit-identical to dequantize-then-fold. */
int tk_linear_salt_seq(tk_ctx *ctx, const tk_salt_desc *layer, const void *act, int act_dtype, size_t m,
                       void *out, int out_dtype);

/* ---- SALT containers: the row sidecar "TSLT" (version 1: dense planes back to back; version 2,
 *      progressive: each plane framed by a tag and a length, residual planes may be sparse) and the sparse
 *      residual plane "TSSP" (crates/tritium-format/src/salt.rs:1-19,229-316,352-434,484-515,596-700;
 *      crates/tritium-format/src/sparse.rs:27-41,92-157,293-309). Host functions; every check of the
 *      reference's readers, in their order, failures are TK_ERR_INVALID_INPUT naming the reference's error.
 *      A sparse plane expands to exactly the dense TQ2_0 row it was made from, so the device path below is
 *      bit-identical whichever way a residual was stored. ---- */
/* packed_salt_row_len: length of the first encoded row in `bytes` (rows are stored back to back) */
int tk_salt_row_len(const uint8_t *bytes, size_t len, size_t *row_len);
/* header fields of the first row: k, plane count, version (any of the three may be NULL) */
int tk_salt_row_info(const uint8_t *bytes, size_t len, size_t *k, size_t *planes, int *version);
/* unpack_salt_row_prefix: `bytes` is exactly one row; all planes are validated, the first
 * min(planes, max_planes) are written as dense TQ2_0 rows of ceil(k/256)*66 bytes, back to back. */
int tk_salt_row_unpack(const uint8_t *bytes, size_t len, size_t max_planes, uint8_t *planes_out,
                       size_t planes_out_len, size_t *k, size_t *n_planes);
/* unpack_sparse_plane + sparse_to_tq2_0: one encoded sparse plane -> its dense TQ2_0 row */
int tk_sparse_plane_to_tq2_0(const uint8_t *bytes, size_t len, uint8_t *row_out, size_t row_out_len, size_t *k);
/* A SALT tensor: n encoded rows back to back (as a bundle stores them) -> up to TK_MAX_PLANES block-scale
 * planes on the device (the loader of crates/tritium-nn/src/layers/packed_salt.rs:612-678). Rows may differ
 * in plane count: plane p of a row with fewer planes is all-zero trits with scale 0 (adds +0.0, as a missing
 * plane adds nothing). max_planes keeps a prefix of every row (the lower-memory tiers of the progressive
 * format). planes_out receives *n_planes buffers (from tk_upload_weights_scaled; free each with
 * tk_free_weights) to put into a tk_salt_desc. A row with more than TK_MAX_PLANES kept planes ->
 * TK_ERR_UNSUPPORTED_FORMAT; a row whose k differs -> TK_ERR_SHAPE_MISMATCH. */
int tk_upload_salt_rows(tk_ctx *ctx, const uint8_t *bytes, size_t len, size_t n, size_t k, size_t max_planes,
                        tk_weights **planes_out, int *n_planes);

/* ---- SALT V2: zero-point-free additive ternary matrices over 256-coefficient allocation tiles with one
 *      to three planes each, f16 scales per group of 128 (or 64) coefficients, three physical codecs
 *      (crates/tritium-format/src/salt_v2.rs:22-32; crates/tritium-format/src/salt_v2_package.rs:38-47). ---- */
enum { TK_SALT_V2_D2 = 0, TK_SALT_V2_B3 = 1, TK_SALT_V2_S34 = 2 }; /* as crates/tritium-cuda/kernels/salt_v2.cu:31-52 */
/* SaltV2Codec::ledger: physical bytes of `trits` logical trits (salt_v2.rs:160-258) */
int tk_salt_v2_payload_bytes(int codec, size_t trits, size_t *bytes);
/* pack_d2 / pack_b3 / pack_s34 and their canonical decoders (salt_v2.rs:268-520): padding slots are zero
 * trits, padding bits zero; reserved codes, B3 bytes >= 243, S34 groups without exactly one zero, wrong
 * lengths are rejected. */
int tk_salt_v2_pack(int codec, const int8_t *trits, size_t n, uint8_t *out, size_t out_len);
int tk_salt_v2_unpack(int codec, const uint8_t *packed, size_t packed_len, size_t n, int8_t *trits);
/* A resident SALT V2 matrix [n,k], in the runtime form the reference's device code takes
 * (crates/tritium-cuda/kernels/salt_v2.cu:114-131; built by crates/tritium-cuda/src/cuda/backend/
 * salt_v2_reader_upload.rs:40-252): `payload` = the codec bytes of every plane, tile after tile, planes of a
 * tile in order (a tile whose planes start at running plane index b has plane j at b*bytes(256) +
 * j*bytes(tile length)); `scales` = one f16 per (plane, scale group) in the same order; plane_counts[tile]
 * in 1..3 (the reference packs the same counts two bits per tile with a rank directory; the adapter hands
 * them over unpacked). Tiles cover the row-major coefficients, tiles == ceil(n*k/256). scale_group is 128 or
 * 64. Host pointers; every plane is decoded once here, so a non-canonical payload is rejected at upload. */
typedef struct tk_salt_v2 tk_salt_v2;
int tk_salt_v2_upload(tk_ctx *ctx, int codec, size_t scale_group, const uint8_t *payload, size_t payload_len,
                      const uint16_t *scales_f16, size_t scale_count, const uint8_t *plane_counts, size_t tiles,
                      size_t n, size_t k, tk_salt_v2 **out);
void tk_salt_v2_free(tk_salt_v2 *t);
/* salt_v2_forward_exact: out[m,n] = act[m,k] x W^T in the reference's pinned scalar order -- per output,
 * segments (tile x scale group) ascending, planes ascending, per plane one f32 accumulator over the columns
 * (add / subtract / skip), ONE multiply by the f16 scale, one add into the output (crates/tritium-cpu/src/
 * salt_v2.rs:10-23,316-423; salt_v2.cu:133-214) -- so the bits are the CPU reference's. The device computes
 * the (segment, plane) terms in parallel and adds them in that order. act and out are device f32. A
 * non-finite activation or result -> TK_ERR_INVALID_INPUT and `out` is left untouched
 * (crates/tritium-cuda/src/cuda/tests.rs:246-280). Synchronizes. */
int tk_salt_v2_forward(tk_ctx *ctx, const tk_salt_v2 *t, const float *act, size_t m, float *out);
/* salt_v2_gather_rows: out[i, :] = row rows[i] of W, each coefficient the f32 sum over its tile's planes,
 * ascending, of +-scale (salt_v2.cu:218-304; crates/tritium-cpu/src/salt_v2.rs:283-300,516-546). rows is a
 * host array (may repeat; order kept); out device f32 [count,k]. A row index >= n -> TK_ERR_INVALID_INPUT. */
int tk_salt_v2_gather_rows(tk_ctx *ctx, const tk_salt_v2 *t, const uint32_t *rows, size_t count, float *out);

/* mpgemm_projected_vjp on device-resident operands (same arithmetic and bits as
 * tk_mpgemm_projected_vjp; precedent for device-resident gradients:
 * crates/tritium-cuda/src/cuda/backend.rs:8755-8830, which stages exactly these buffers). scales [n],
 * act [m,k], grad_output [m,n], grad_act [m,k], grad_w [n,k], grad_bias [n], all f32 on ctx's
 * device; any of the three outputs may be NULL and is then skipped (act is only read for grad_w).
 * Enqueued on ctx's stream, not synchronised. */
int tk_projected_vjp(tk_ctx *ctx, const tk_weights *weights, const float *scales, const float *act,
                     const float *grad_output, size_t m, float *grad_act, float *grad_w,
                     float *grad_bias);

/* Reference-order float contraction: one thread per output, a single f32 accumulator walked in k
 * order (crates/tritium-core/src/reference.rs:25-54) — bit-identical to the CPU backend for any
 * float input, NaN/Inf included. Slow; kept as the exact fallback and as a cross-check. */
int tk_linear_float_seq(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype,
                        size_t m, void *out, int out_dtype);

/* Several independent linears in ONE launch (q/k/v or gate/up sharing a step; or a whole stack of
 * projections whose inputs are already known). All members must share act_dtype, out_dtype, the
 * mode and the plane count. Build once, launch many times. */
typedef struct tk_group tk_group;
typedef struct tk_group_member {
  tk_linear_desc layer;
  const void *act;  /* [m,k] */
  size_t m;
  void *out;        /* [m,n] */
} tk_group_member;
typedef enum tk_group_mode { TK_GROUP_FLOAT = 0, TK_GROUP_A8 = 1 } tk_group_mode;
int tk_group_create(tk_ctx *ctx, const tk_group_member *members, size_t count, int mode,
                    int act_dtype, int out_dtype, tk_group **out);
/* A W1.58A8 group whose members read RMSNorm(act): norms[i] belongs to members[i]; an entry with a
 * null weight leaves that member's activation as it is. Members that share activation and norm
 * share one normalization + quantization (q/k/v after the attention norm, gate/up after the FFN
 * norm: crates/tritium-cuda/src/cuda/mod.rs:1029-1064). */
int tk_group_create_normed(tk_ctx *ctx, const tk_group_member *members, const tk_rmsnorm *norms, size_t count,
                           int act_dtype, int out_dtype, tk_group **out);
int tk_group_launch(tk_ctx *ctx, tk_group *group);
/* The two launches of a group separately (activation prep, then the contraction), so a harness can
 * bracket the contraction kernel alone with events. tk_group_launch == parts(1, 1). */
int tk_group_launch_parts(tk_ctx *ctx, tk_group *group, int do_prep, int do_main);
void tk_group_destroy(tk_group *group);

/* GEMV -> GEMM crossover in activation rows; the reference's knob is TRITIUM_IMMA_MIN_M, default
 * 32, integer >= 2 (crates/tritium-cuda/src/cuda/backend.rs:6861-6876). The environment variable
 * TRITIUM_MI355X_GEMM_MIN_M is read at tk_init with the same loud-reject rule. */
int tk_set_gemm_min_m(tk_ctx *ctx, int min_m);
int tk_get_gemm_min_m(const tk_ctx *ctx);

/* Force one decode kernel for every later launch: 0 automatic, 1 K-split, 2 streaming (K passes
 * through LDS), 3 flow (all of K resident in LDS; falls back to 2 when it does not fit). All give
 * identical bits; the knob exists for tests and tuning. */
int tk_set_decode_kernel(tk_ctx *ctx, int variant);
/* Consecutive output tiles a wave of the flow kernel walks as one stream; 0 = chosen from the size
 * of the launch. A tuning knob: results do not depend on it. */
int tk_set_flow_run_tiles(tk_ctx *ctx, int tiles);
/* Positions in the flow kernel's prefetch ring: 0 = chosen per launch (fewest padded positions for
 * the K block counts of the launch), or 2..5. A tuning knob: results do not depend on it. */
int tk_set_flow_ring(tk_ctx *ctx, int positions);
/* Matrix instruction of the flow kernel for 17..64 operand rows and one or two planes: 0 = chosen
 * per launch (32x32x32 for 25..32 rows that take at most 64 KiB of LDS), 16 = always 16x16x64,
 * 32 = 32x32x32 wherever its operand rows fit in LDS. A tuning and test knob: both forms give
 * identical bits. */
int tk_set_flow_mfma(tk_ctx *ctx, int rows);
/* Output tiles per wave of the one-plane prefill kernel: 0 = chosen per launch (4, or 2 when 4 would
 * leave fewer than four workgroups per CU), 2 or 4 to force. A tuning and test knob: both forms give
 * identical bits. */
int tk_set_gemm_tiles(tk_ctx *ctx, int tiles);
/* The 64 x 128 form of the one-plane prefill kernel has its four waves side by side (64 rows x 32 outputs
 * each). on != 0 arranges them two by two (32 rows x 64 outputs each: half the LDS reads, twice the weight
 * loads; measured 3-6% slower, identical bits). A measurement knob. */
int tk_set_gemm_two_by_two(tk_ctx *ctx, int on);
/* Activation prep (quantization / digit split): launches of up to `rows` tokens give every token a whole
 * workgroup instead of one wave (few tokens: the launch lasts as long as one token's chain of instructions).
 * Default 384 (the digit split of the float contract: 8/3 of it). Process-wide; identical bits either way. A tuning and test knob. */
int tk_set_prep_team_rows(tk_ctx *ctx, int rows);
/* Host-slice calls (tk_mpgemm, tk_mpgemm_with_act_quant) whose operands (activation, scales, output) total at most
 * `bytes` go through a pinned host block that the context owns: one copy kernel brings activation and scales to the
 * device, the kernels write the output into the block, the call synchronizes once -- in place of four transfers from
 * and to pageable memory. Larger calls, and when no pinned memory can be had, take those transfers. Default 1 MiB;
 * 0 = never; at most 64 MiB. Identical results. A tuning and test knob. */
int tk_set_host_direct_bytes(tk_ctx *ctx, size_t bytes);
/* Decode calls of very few tokens run as ONE launch: the decode kernel quantizes (or digit-splits) the tokens
 * itself, every workgroup for itself, instead of a prep launch in front of it. Single calls (tk_linear_a8,
 * tk_linear_float, tk_linear_a8_residual; tk_linear_rmsnorm_a8 for one token, norm included) and groups created
 * after the call (every member within the limits; a member behind an RMSNorm holds one token). Limits: K a multiple
 * of 256 up to 8192, 16-byte aligned f32 or bf16 rows (and norm weights), operand rows within 62 KiB of LDS in the
 * flow kernel or 48 KiB in the K-split kernel of narrow launches, and there at most eight output tiles per CU (a
 * workgroup takes up to four behind one quantization). tokens: -1 (default) = one token, or two under
 * the int8 contract in the K-split kernel; 0 = never; 1..4 = up to that many. Identical bits either way. A tuning
 * and test knob. */
int tk_set_fuse_tokens(tk_ctx *ctx, int tokens);
/* Calls of this context so far that ran in that single-launch form (for tests of the dispatch). */
int tk_get_fused_calls(tk_ctx *ctx, unsigned long long *count);
/* Name of the contraction kernel the last single call of this context (tk_linear_*, tk_mpgemm*) took:
 * "flow", "flow32", "flow3", "stream", "ksplit_decode", "gemm64", "gemm64_ksplit", "gemm128", "gemm256";
 * "" before the first call. A static string. For tests of the dispatch; no counterpart in the reference. */
const char *tk_last_kernel(tk_ctx *ctx);
/* Row count of the workgroup tile for single launches of one plane under the int8 contract (f32 or bf16
 * rows of whole 16-byte pieces at a 16-byte aligned address, no residual): 0 = chosen per launch, 64 = the
 * 64-row kernels, 128 = the 128 x 256 kernel, which shares both operands through LDS, 256 = the 256-row kernel,
 * which expands the weight tile to int8 once per workgroup, in LDS. Other launches take the 64-row kernels
 * whatever this says. A tuning and test knob: identical bits. */
int tk_set_gemm_rows(tk_ctx *ctx, int rows);
/* Form of the 256-row kernel: 0 = four waves of 64 rows over a column block of 224 outputs, one workgroup per CU; 1 =
 * eight waves of 32 rows; 2 = four waves over a part of the column block (128 or 96 outputs), two workgroups per CU;
 * -1 (the state of a new context) = form 1, the one the automatic dispatch uses (for launches of 0.7 .. 1 workgroups per
 * CU). A measurement and test knob: identical bits. */
int tk_set_gemm256_form(tk_ctx *ctx, int form);
/* A grouped launch whose members partly fit LDS runs two kernels (the flow kernel for those that fit, the prefill
 * kernel for the others). on != 0 (default): side by side on two streams of the context, joined before
 * anything enqueued later; 0: one after the other. A measurement knob: identical results. */
int tk_set_group_overlap(tk_ctx *ctx, int on);
/* K slices of the prefill kernel in single launches: 0 = chosen per launch (a launch with fewer
 * workgroups than CUs is cut into about one workgroup per CU, at least two K blocks per slice), 1 =
 * never split, 2..64 = that many slices where K allows. Integer partial sums, added by the last
 * workgroup to arrive: identical bits. A tuning and test knob. */
int tk_set_gemm_ksplit(tk_ctx *ctx, int slices);
/* The K-split decode kernel has the finer grain (a single narrow layer), the streaming and flow
 * kernels walk whole output tiles per wave (launches that fill the chip): the latter are taken when
 * a launch needs at least this many workgroups; default = the device's CU count. No counterpart
 * in the reference; results do not depend on it. */
int tk_set_stream_min_groups(tk_ctx *ctx, int groups);
int tk_get_stream_min_groups(const tk_ctx *ctx);

/* tk_mpgemm answers float problems of at most this many multiply-accumulates (m·n·k; default 2^20,
 * the largest conformance vector, crates/tritium-testkit/src/generate.rs:203-214) with the
 * reference-order kernel of tk_linear_float_seq: such calls are latency-bound either way, and the
 * result is then bit-identical to the CPU backend rather than merely within its 1e-4 tolerance.
 * 0 sends every float call to the MFMA path. */
int tk_set_exact_max_macs(tk_ctx *ctx, size_t macs);
size_t tk_get_exact_max_macs(const tk_ctx *ctx);

/* ---- plumbing: device memory, stream, events (what the harness and a backend crate need; the
 *      reference's device backends own the same privately: crates/tritium-rocm/src/rocm.rs:84-174
 *      device buffers, :207-242 stream and synchronous calls) ---- */
int tk_malloc(tk_ctx *ctx, size_t bytes, void **dptr);
int tk_free(tk_ctx *ctx, void *dptr);
int tk_memcpy_h2d(tk_ctx *ctx, void *dst, const void *src, size_t bytes);
int tk_memcpy_d2h(tk_ctx *ctx, void *dst, const void *src, size_t bytes);
int tk_memset(tk_ctx *ctx, void *dst, int value, size_t bytes);
int tk_sync(tk_ctx *ctx);
/* The hipStream_t the context launches on. Once a call of the same shapes has run, a device-resident linear or
 * group call enqueues kernels and event waits only (no allocation, no synchronisation, no memset), so a caller may
 * capture this stream around such calls and replay the graph. */
void *tk_stream(tk_ctx *ctx);
typedef struct tk_event tk_event;
int tk_event_create(tk_ctx *ctx, tk_event **out);
int tk_event_record(tk_ctx *ctx, tk_event *ev);
int tk_event_elapsed_ms(tk_event *start, tk_event *stop, float *ms); /* waits for `stop` */
void tk_event_destroy(tk_event *ev);
/* A plain device-to-device copy kernel of `bytes` bytes (multiple of 16), used to calibrate
 * hardware traffic counters against a known size. */
int tk_copy_kernel(tk_ctx *ctx, void *dst, const void *src, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif
