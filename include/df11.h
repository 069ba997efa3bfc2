/*
 * df11.h -- C-ABI of the MI355X (gfx950) DFloat11 weight-decompression path.
 *
 * Two shared libraries export these symbols:
 *   libdf11_hip.so    device entry points (section "Device"), needs the HIP runtime
 *   libdf11_codec.so  host-only codec (section "Host codec"), plain C++
 *
 * Conventions: every function returns DF11_OK (0) or a negative DF11_ERR_*
 * code; df11_error_string() names it.  The library never allocates or frees
 * device memory: kernels are enqueued on the caller's stream and the caller owns
 * every buffer until that work completes (df11_decode_static_workspace keeps its
 * workspace in a fixed device array of the library instead).  Only df11_prepare (load time) may
 * wait for the stream; df11_decode never synchronises.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).
 */
#ifndef DF11_H
#define DF11_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DF11_OK 0
#define DF11_ERR_INVALID_ARGUMENT (-1)
#define DF11_ERR_UNSUPPORTED (-2)
#define DF11_ERR_HIP (-3)           /* a HIP runtime call failed; see df11_last_hip_error() */
#define DF11_ERR_CAPACITY (-4)      /* a buffer is too small, or the input exceeds a fixed capacity */
#define DF11_ERR_FORMAT (-5)        /* the code cannot be expressed in the DF11 LUT layout */

/* Format constants (reference: dfloat11/dfloat11.py:45-46). */
#define DF11_BYTES_PER_THREAD 8
#define DF11_THREADS_PER_BLOCK 512
#define DF11_BLOCK_BYTES 4096
#define DF11_GAP_BYTES_PER_BLOCK 320
#define DF11_MAX_ELEMS_PER_BLOCK 32768
#define DF11_SUBBLOCK_BYTES 512
#define DF11_MAX_ELEMS_PER_SUBBLOCK 4096

/* Version of this interface: 5 = df11_decode_rows and DF11_PLAN_PORTABLE added
 * (4 = df11_decode_with_plan replaces the process-wide df11_force_launch_plan,
 * df11_calibration_copy removed; 3 = df11_decode_static_workspace and
 * df11_launch_plan_name added, workspace holds fused LUT rows). */
int df11_version(void);
const char *df11_error_string(int code);

/* ------------------------------------------------------------------ Device */

/* Text of the last HIP error seen by this library on the calling thread. */
const char *df11_last_hip_error(void);

/*
 * Size in bytes of the decode workspace of a stream with n_bytes bytes of
 * encoded_exponent: a 64-byte header, the multi-symbol decode tables derived
 * from `luts`, and the output index at which each 512-byte sub-block of the
 * bitstream starts (4 bytes per sub-block, about 0.2 % of the compressed size).
 */
size_t df11_workspace_bytes(int64_t n_bytes);

/*
 * Fill the workspace of one compressed tensor.  Everything in it depends only on
 * the compressed stream, so this runs once per tensor at load time; the
 * reference's closest counterpart is the load-time derivation of shared_mem_size
 * from output_positions (dfloat11/dfloat11.py:299-306).
 *   luts, encoded_exponent, output_positions, gaps   as for df11_decode (device)
 *   workspace   device, df11_workspace_bytes(n_bytes) bytes, 16-byte aligned
 *   max_elems_per_subblock   host out, may be NULL: the largest number of
 *               elements any 512-byte sub-block produces; pass it to df11_decode.
 *               When non-NULL the call waits for `stream` (load time only).
 */
int df11_prepare(const uint8_t *luts, const uint8_t *encoded_exponent,
                 const uint32_t *output_positions, const uint8_t *gaps,
                 int32_t n_luts, int64_t n_bytes, int64_t n_elements,
                 void *workspace, int32_t *max_elems_per_subblock, void *stream);

/*
 * Decode one DF11 stream into BF16.  Replaces the reference's kernel launch
 *   _decode(grid, block, shared_mem, args=[luts, encoded_exponent, sign_mantissa,
 *           output_positions, gaps, reconstructed, n_luts, n_bytes, n_elements])
 * (dfloat11/dfloat11.py:139-151; kernel signature dfloat11/decode.cu:25-34).
 * The six pointers and three sizes keep the reference's order and meaning;
 * sizes are 64-bit here.  All pointers are device pointers.  Asynchronous on
 * `stream`; allocates nothing.
 *   output_positions  u32[ceil(n_bytes/4096)] at least; only df11_prepare reads
 *                     it, the decode uses the finer positions in the workspace
 *   gaps              u8[320 * ceil(n_bytes/4096)]
 *   workspace         filled by df11_prepare for the same stream
 *   max_elems_per_subblock  as returned by df11_prepare (it sizes the LDS
 *                     staging, the role shared_mem_size plays in the reference);
 *                     <= 0 selects the format's worst case (4096)
 */
int df11_decode(const uint8_t *luts, const uint8_t *encoded_exponent, const uint8_t *sign_mantissa,
                const uint32_t *output_positions, const uint8_t *gaps, uint16_t *outputs,
                int32_t n_luts, int64_t n_bytes, int64_t n_elements,
                const void *workspace, int32_t max_elems_per_subblock, void *stream);

/*
 * df11_decode for some rows of the output only: the stream decodes to a matrix of
 * row_elements elements per row, and only the 512-byte pieces of bitstream that hold
 * elements of rows row_ids[0 .. n_ids) are decoded, into the same places of `outputs`
 * (the full-size buffer) that df11_decode writes them to.  Every such piece is written
 * out whole, so up to a piece's worth of elements before and after a row are decoded
 * with it; every other element of `outputs` is left as it was.  For an embedding,
 * whose forward pass reads the rows it looks up and nothing else (reference:
 * dfloat11.py:155-157 decodes the whole table before every lookup).
 *   row_ids     DEVICE pointer to n_ids row numbers (int64, 8-byte aligned), read by
 *               the kernel in stream order: the caller need not know them.  Numbers
 *               outside the matrix select nothing; repeated ones cost repeated work.
 * Other arguments and return codes as for df11_decode; DF11_ERR_UNSUPPORTED where only
 * DF11_PLAN_PORTABLE can run (decode the whole stream there).  The work is
 * proportional to n_ids, with a search per id on top: beyond a quarter of the rows or
 * so, df11_decode is the faster call.
 */
int df11_decode_rows(const uint8_t *luts, const uint8_t *encoded_exponent, const uint8_t *sign_mantissa,
                     const uint32_t *output_positions, const uint8_t *gaps, uint16_t *outputs,
                     int32_t n_luts, int64_t n_bytes, int64_t n_elements, const void *workspace,
                     int32_t max_elems_per_subblock, void *stream, const int64_t *row_ids,
                     int64_t n_ids, int64_t row_elements);

/*
 * df11_prepare + df11_decode in one call, with the workspace in a device array
 * that the library itself holds (DF11_STATIC_WORKSPACE_BYTES on every GPU the
 * library's code is loaded on, from that load until the process ends, whether
 * this entry point is ever called or not).  No counterpart in
 * the reference: it is for callers that cannot allocate device memory or wait
 * for the device -- code under HIP graph capture, serving loops, harnesses that
 * forbid hipMalloc.  The call allocates and frees nothing, never synchronises,
 * and enqueues three kernels on `stream` (tables, sub-block positions, decode).
 * Arguments as for df11_decode, without the workspace.
 *   max_elems_per_subblock  an upper bound on the elements any 512-byte
 *               sub-block produces, if the caller knows one (it sizes the LDS
 *               staging; too small a bound truncates sub-blocks); <= 0 selects
 *               the format's worst case (4096), which is always safe
 * Streams of more than DF11_STATIC_MAX_STREAM_BYTES bytes of encoded_exponent
 * are rejected with DF11_ERR_CAPACITY.  All calls on one GPU share the one
 * array: calls that overlap in time on the same GPU (different streams, or a
 * captured graph replayed on one stream while an eager call runs on another)
 * race and corrupt each other's output without an error; the caller orders
 * them, with an event between streams where they differ.  The first call on a
 * GPU looks the array's device
 * address up (hipGetSymbolAddress); make that call outside a graph capture.
 */
#define DF11_STATIC_WORKSPACE_BYTES 4194304
#define DF11_STATIC_MAX_STREAM_BYTES 533385216   /* 130221 bitstream blocks */
int df11_decode_static_workspace(const uint8_t *luts, const uint8_t *encoded_exponent,
                                 const uint8_t *sign_mantissa, const uint32_t *output_positions,
                                 const uint8_t *gaps, uint16_t *outputs, int32_t n_luts,
                                 int64_t n_bytes, int64_t n_elements,
                                 int32_t max_elems_per_subblock, void *stream);

/*
 * df11_decode with the launch plan chosen by the caller.  The decode kernel is
 * compiled for three launch plans (workgroups resident per CU and how far ahead
 * it requests sign_mantissa bytes: DF11_PLAN_WIDE, _DEEP, _DEEPEST; the two plans
 * for large streams come in further compilations that differ in how wavefront
 * priorities are set and in the cache policy of the loads, and `wide` in two more
 * with four workgroups per CU, which the stream's size and code lengths decide
 * when the plan is left to the library), nine kernels in all with
 * DF11_PLAN_PORTABLE.  df11_decode picks the plan per stream from its size and
 * its elements per 512 bytes of bitstream; this entry point takes it as an
 * argument, for tests that drive every stream through every plan and for
 * measurements.  DF11_PLAN_AUTO behaves as df11_decode does.  The choice is local
 * to the call: nothing in the library remembers it.  No counterpart in the
 * reference; every plan decodes every stream to the same bits.
 */
#define DF11_PLAN_AUTO (-1)
#define DF11_PLAN_WIDE 0
#define DF11_PLAN_DEEP 1
#define DF11_PLAN_DEEPEST 2
/* `wide` with workgroup memory addressed through its symbol instead of from a constant:
 * what every stream runs, whatever plan is asked for, if a toolchain gives the other
 * kernels workgroup memory of its own (checked once per device); about 13 % more vector
 * instructions. */
#define DF11_PLAN_PORTABLE 3
int df11_decode_with_plan(const uint8_t *luts, const uint8_t *encoded_exponent,
                          const uint8_t *sign_mantissa, const uint32_t *output_positions,
                          const uint8_t *gaps, uint16_t *outputs, int32_t n_luts, int64_t n_bytes,
                          int64_t n_elements, const void *workspace,
                          int32_t max_elems_per_subblock, void *stream, int32_t plan);

/*
 * Which compilation of the decode kernel df11_decode launches for a stream of
 * n_bytes of encoded_exponent and n_elements on a device of compute_units CUs
 * (when the LDS the stream needs leaves room for the plan's workgroups per CU):
 * "wide", "wide/full", "wide/dense", "deep", "deep/short", "deep/small", "deepest"
 * or "deepest/short";
 * "" for sizes that are not positive.  Needs no GPU.  Testing aid with no
 * counterpart in the reference.
 */
const char *df11_launch_plan_name(int64_t n_bytes, int64_t n_elements, int32_t compute_units);

/* -------------------------------------------------------------- Host codec */

/*
 * Exponent histogram of n BF16 words: hist[e] = #{ i : (w[i] >> 7) & 0xFF == e }.
 * Replaces the histogram half of get_codec (dfloat11_utils.py:24-30).
 */
int df11_histogram(const uint16_t *w, int64_t n, uint64_t hist[256], int32_t n_threads);

/*
 * Prefix code for the exponent bytes: optimal (Huffman) including one
 * end-of-stream leaf of weight 1, limited to 32 bits, and shaped so that the
 * DF11 LUT layout can express it (at most 16 sub-tables; symbols >= 240 only
 * on the fourth LUT level).  code_len[s] == 0 for absent symbols.
 * Replaces HuffmanCodec.from_frequencies + get_32bit_codec
 * (dfloat11_utils.py:32, 37-65).
 */
int df11_build_code(const uint64_t hist[256], uint8_t code_len[256], uint32_t code_val[256],
                    int32_t *eof_len, uint32_t *eof_val);

/*
 * Hierarchical byte LUTs + length row for a code (get_luts,
 * dfloat11_utils.py:68-115).  luts has room for cap_rows rows of 256 bytes;
 * *n_luts receives the row count (decode rows + 1).
 */
int df11_build_luts(const uint8_t code_len[256], const uint32_t code_val[256],
                    uint8_t *luts, int32_t cap_rows, int32_t *n_luts);

/* Split BF16 words into exponent bytes and sign|mantissa bytes (dfloat11_utils.py:175-178). */
int df11_split(const uint16_t *w, int64_t n, uint8_t *exponent, uint8_t *sign_mantissa,
               int32_t n_threads);

/*
 * Sizes of the encoded stream for `n` exponent bytes under a code:
 * n_bytes (encoded_exponent), n_blocks = ceil(n_bytes/4096).
 */
int df11_encode_size(const uint8_t *exponent, int64_t n, const uint8_t code_len[256],
                     int64_t *n_bytes, int64_t *n_blocks, int32_t n_threads);

/*
 * Bit-pack the exponent bytes MSB-first and emit the per-thread gaps and
 * per-block output positions (encode, dfloat11_utils.py:118-170).
 *   encoded           u8[n_bytes]            from df11_encode_size
 *   gaps              u8[320 * n_blocks]
 *   output_positions  u32[n_blocks + 1]      always n_blocks + 1 entries
 * The final partial byte is padded with the leading bits of the end-of-stream
 * code, as the reference does.
 */
int df11_encode(const uint8_t *exponent, int64_t n, const uint8_t code_len[256],
                const uint32_t code_val[256], int32_t eof_len, uint32_t eof_val,
                uint8_t *encoded, int64_t n_bytes, uint8_t *gaps, uint32_t *output_positions,
                int64_t n_blocks, int32_t n_threads);

#ifdef __cplusplus
}
#endif
#endif /* DF11_H */
