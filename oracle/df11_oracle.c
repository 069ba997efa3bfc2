/*
 * df11_oracle.c -- TEST INFRASTRUCTURE ONLY.
 *
 * Scalar CPU restatement of the DFloat11 reference algorithm for the weight
 * decompression path.  It exists to CHECK the HIP path; nothing that ships may
 * call it.  Only tests, the smoke check and the cpu_baseline leg of the
 * benchmark load this library.
 *
 * The reference has no CPU decoder: its only decoder is the CUDA kernel
 * dfloat11/decode.cu.  df11o_decode_blocks() below follows that kernel thread
 * by thread (same 12-byte fetch, same 5-bit gap, same two passes around an
 * exclusive prefix sum, same staging buffer and clamps).  df11o_encode()
 * follows the Python bit packer dfloat11/dfloat11_utils.py:118-170 statement
 * by statement, quirks included.  df11o_decode_sequential() is an independent
 * second opinion that ignores gaps and positions altogether.
 *
 * Pinning status (the reference holds no golden vectors for this path):
 *   df11o_split / df11o_merge  : closed form, exhaustive over 65536 patterns.
 *   df11o_encode               : hand-packed streams + the pure-Python
 *                                restatement in df11_oracle.py + invariants.
 *   df11o_decode_blocks        : identity decode(encode(W)) == W, agreement
 *                                with df11o_decode_sequential, hand-packed
 *                                streams.
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define BYTES_PER_THREAD 8      /* dfloat11.py:45 */
#define N_THREADS 512           /* dfloat11.py:46 */
#define BLOCK_BYTES (BYTES_PER_THREAD * N_THREADS)

#define DF11O_OK 0
#define DF11O_ERR_ARG (-1)
#define DF11O_ERR_ZERO_LEN (-2)   /* a decoded symbol has code length 0: the reference kernel would spin forever */
#define DF11O_ERR_LUT_OOB (-3)    /* a pointer entry names a LUT row the tensor does not have */
#define DF11O_ERR_STAGE_OOB (-4)  /* a thread writes past the staging buffer the reference would have allocated */
#define DF11O_ERR_CAPACITY (-5)

/* dfloat11_utils.py:175-178: W viewed as int16;
 * exponent = (W >> 7) & 0xFF ; sign_mantissa = ((W >> 8) & 0x80) | (W & 0x7F) */
void df11o_split(const uint16_t *w, int64_t n, uint8_t *exponent, uint8_t *sign_mantissa)
{
    for (int64_t i = 0; i < n; ++i) {
        int16_t v = (int16_t)w[i];
        exponent[i] = (uint8_t)((v >> 7) & 0xFF);
        sign_mantissa[i] = (uint8_t)(((v >> 8) & 0x80) | (v & 0x7F));
    }
}

/* decode.cu:207-210: high byte = (sm & 128) | (exp >> 1); low byte = (exp << 7) | (sm & 127) */
static inline uint16_t merge_one(uint8_t exponent, uint8_t sm)
{
    uint8_t hi = (uint8_t)((sm & 128) | (exponent >> 1));
    uint8_t lo = (uint8_t)((exponent << 7) | (sm & 127));
    return (uint16_t)((hi << 8) | lo);
}

void df11o_merge(const uint8_t *exponent, const uint8_t *sign_mantissa, int64_t n, uint16_t *w)
{
    for (int64_t i = 0; i < n; ++i) w[i] = merge_one(exponent[i], sign_mantissa[i]);
}

/* decode.cu:105-113: root lookup on the top byte, then up to three more
 * levels; any value >= 240 on levels 0..2 names row (256 - value); the fourth
 * level is taken as a symbol without testing it. */
static inline int lut_walk(const uint8_t *luts, int n_luts, uint64_t window, uint8_t *symbol)
{
    uint8_t d = luts[window >> 56];
    for (int level = 1; level <= 3 && d >= 240; ++level) {
        int row = 256 - d;
        if (row >= n_luts) return DF11O_ERR_LUT_OOB;
        d = luts[256 * row + ((window >> (56 - 8 * level)) & 0xff)];
    }
    *symbol = d;
    return DF11O_OK;
}

static inline uint8_t fetch(const uint8_t *codes, int64_t n_bytes, int64_t i)
{
    /* decode.cu:42-77 guards every byte load with i < n_bytes; the shipped
     * PTX zero-initialises the registers (decode.ptx:53-54). */
    return i < n_bytes ? codes[i] : 0;
}

typedef struct {
    uint8_t bytes[12];
    uint8_t gap;
} thread_in;

static void thread_fetch(const uint8_t *codes, const uint8_t *gaps, int64_t n_gap_bytes,
                         int64_t n_bytes, int64_t gid, thread_in *t)
{
    for (int k = 0; k < 12; ++k) t->bytes[k] = fetch(codes, n_bytes, gid * BYTES_PER_THREAD + k);
    /* decode.cu:85-87; the byte after the last gap byte is read by the last
     * thread of the grid but never contributes (shift is 8 there). */
    int64_t gi = gid * 5 / 8;
    uint16_t pair = (uint16_t)((gaps[gi] << 8) | (gi + 1 < n_gap_bytes ? gaps[gi + 1] : 0));
    t->gap = (uint8_t)((pair >> (11 - (gid * 5 % 8))) & 0x1f);
}

static inline uint64_t be64(const uint8_t *b)
{
    uint64_t v = 0;
    for (int k = 0; k < 8; ++k) v = (v << 8) | b[k];
    return v;
}

static inline uint32_t be32(const uint8_t *b)
{
    return ((uint32_t)b[0] << 24) | ((uint32_t)b[1] << 16) | ((uint32_t)b[2] << 8) | b[3];
}

/* Pass 1, decode.cu:89-144: count the codes that start inside the 64-bit chunk. */
static int thread_count(const uint8_t *luts, int n_luts, const thread_in *t, uint32_t *count)
{
    const uint8_t *lens = luts + 256 * (n_luts - 1);
    uint64_t window = be64(t->bytes) << t->gap;
    unsigned free_bits = t->gap;
    uint32_t n = 0;
    uint8_t sym;
    int rc;
    while (free_bits < 32) {
        if ((rc = lut_walk(luts, n_luts, window, &sym))) return rc;
        n += 1;
        uint8_t len = lens[sym];
        if (len == 0) return DF11O_ERR_ZERO_LEN;
        window <<= len;
        free_bits += len;
    }
    window |= (uint64_t)be32(t->bytes + 8) << (free_bits - 32);
    free_bits -= 32;
    while (4 + free_bits / 8 < BYTES_PER_THREAD) {
        if ((rc = lut_walk(luts, n_luts, window, &sym))) return rc;
        n += 1;
        uint8_t len = lens[sym];
        if (len == 0) return DF11O_ERR_ZERO_LEN;
        window <<= len;
        free_bits += len;
    }
    *count = n;
    return DF11O_OK;
}

/* Pass 2, decode.cu:180-247: decode again and write merged BF16 words into the
 * block's staging buffer at (output_idx - block base). */
static int thread_emit(const uint8_t *luts, int n_luts, const thread_in *t,
                       const uint8_t *sign_mantissa, uint32_t output_idx, uint32_t end_output_idx,
                       uint32_t write_offset, uint16_t *stage, int64_t stage_cap)
{
    const uint8_t *lens = luts + 256 * (n_luts - 1);
    uint64_t window = be64(t->bytes) << t->gap;
    unsigned free_bits = t->gap;
    uint8_t sym;
    int rc;
    while (free_bits < 32 && output_idx < end_output_idx) {
        if ((rc = lut_walk(luts, n_luts, window, &sym))) return rc;
        if ((int64_t)(output_idx - write_offset) >= stage_cap) return DF11O_ERR_STAGE_OOB;
        stage[output_idx - write_offset] = merge_one(sym, sign_mantissa[output_idx]);
        output_idx += 1;
        uint8_t len = lens[sym];
        if (len == 0) return DF11O_ERR_ZERO_LEN;
        window <<= len;
        free_bits += len;
    }
    /* The reference refills unconditionally (decode.cu:222-228); when the
     * first loop stopped early on output_idx the second loop does not run, so
     * the refill only matters when free_bits >= 32. */
    if (free_bits >= 32) {
        window |= (uint64_t)be32(t->bytes + 8) << (free_bits - 32);
        free_bits -= 32;
    }
    while (output_idx < end_output_idx) {
        if ((rc = lut_walk(luts, n_luts, window, &sym))) return rc;
        if ((int64_t)(output_idx - write_offset) >= stage_cap) return DF11O_ERR_STAGE_OOB;
        stage[output_idx - write_offset] = merge_one(sym, sign_mantissa[output_idx]);
        output_idx += 1;
        uint8_t len = lens[sym];
        if (len == 0) return DF11O_ERR_ZERO_LEN;
        window <<= len;
        free_bits += len;
    }
    return DF11O_OK;
}

/*
 * Restatement of one launch of `decode` (decode.cu:25-253) restricted to the
 * thread blocks [block_begin, block_end).  Arguments keep the kernel's order.
 * `n_positions` is the number of u32 entries in position_offsets; the
 * reference reads entry block+1 without a bound (decode.cu:176) -- here a
 * missing entry reads as n_elements, which is what the clamp at decode.cu:250
 * makes of it.  `stage_elems` is the staging capacity the reference derives at
 * load time, max(diff(position_offsets)) (dfloat11.py:301-306); pass <= 0 to
 * have it computed here.
 */
int df11o_decode_blocks(const uint8_t *luts, const uint8_t *codes, const uint8_t *sign_mantissa,
                        const uint32_t *position_offsets, const uint8_t *gaps, uint16_t *outputs,
                        int n_luts, int64_t n_bytes, int64_t n_elements, int64_t n_positions,
                        int64_t block_begin, int64_t block_end, int64_t stage_elems)
{
    if (n_luts < 2 || n_bytes < 0 || n_elements < 0 || n_positions < 1) return DF11O_ERR_ARG;
    int64_t n_blocks = (n_bytes + BLOCK_BYTES - 1) / BLOCK_BYTES;
    if (block_begin < 0 || block_end > n_blocks) return DF11O_ERR_ARG;
    int64_t n_gap_bytes = n_blocks * (N_THREADS * 5 / 8);
    if (stage_elems <= 0) {
        stage_elems = 0;
        for (int64_t b = 0; b + 1 < n_positions; ++b) {
            int64_t d = (int64_t)position_offsets[b + 1] - (int64_t)position_offsets[b];
            if (d > stage_elems) stage_elems = d;
        }
    }
    uint16_t *stage = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(stage_elems > 0 ? stage_elems : 1));
    thread_in *tin = (thread_in *)malloc(sizeof(thread_in) * N_THREADS);
    uint32_t counts[N_THREADS];
    int rc = DF11O_OK;
    for (int64_t block = block_begin; block < block_end && rc == DF11O_OK; ++block) {
        uint32_t base = block < n_positions ? position_offsets[block] : (uint32_t)n_elements;
        uint32_t next = block + 1 < n_positions ? position_offsets[block + 1] : (uint32_t)n_elements;
        for (int t = 0; t < N_THREADS; ++t) {
            thread_fetch(codes, gaps, n_gap_bytes, n_bytes, block * N_THREADS + t, &tin[t]);
            if ((rc = thread_count(luts, n_luts, &tin[t], &counts[t]))) break;
        }
        if (rc) break;
        /* decode.cu:146-178: exclusive prefix sum seeded with the block base. */
        uint32_t running = base;
        for (int t = 0; t < N_THREADS; ++t) {
            uint32_t output_idx = running;
            running += counts[t];
            /* decode.cu:181 */
            uint32_t end_idx = output_idx + counts[t];
            if ((int64_t)end_idx > n_elements) end_idx = (uint32_t)n_elements;
            if ((rc = thread_emit(luts, n_luts, &tin[t], sign_mantissa, output_idx, end_idx, base,
                                  stage, stage_elems))) break;
        }
        if (rc) break;
        /* decode.cu:248-252 */
        int64_t lim = (int64_t)next - base;
        if (n_elements - (int64_t)base < lim) lim = n_elements - (int64_t)base;
        for (int64_t i = 0; i < lim; ++i) outputs[i + base] = stage[i];
    }
    free(tin);
    free(stage);
    return rc;
}

/*
 * Independent sequential decoder: starts at bit 0 and walks the whole stream,
 * ignoring gaps and position_offsets.  Uses a plain bit reader over the
 * length/codeword table (not the byte LUTs), so it shares no lookup logic with
 * df11o_decode_blocks.  code_len[s]==0 means symbol s is absent.
 */
int df11o_decode_sequential(const uint8_t *code_len, const uint32_t *code_val,
                            const uint8_t *codes, int64_t n_bytes,
                            const uint8_t *sign_mantissa, int64_t n_elements, uint16_t *outputs)
{
    int64_t bit = 0, total_bits = n_bytes * 8;
    for (int64_t i = 0; i < n_elements; ++i) {
        uint32_t acc = 0;
        int len = 0, found = -1;
        while (found < 0) {
            if (bit >= total_bits || len >= 32) return DF11O_ERR_ARG;
            acc = (acc << 1) | ((codes[bit >> 3] >> (7 - (bit & 7))) & 1);
            ++bit; ++len;
            for (int s = 0; s < 256; ++s)
                if (code_len[s] == len && code_val[s] == acc) { found = s; break; }
        }
        outputs[i] = merge_one((uint8_t)found, sign_mantissa[i]);
    }
    return DF11O_OK;
}

/*
 * Restatement of encode() (dfloat11_utils.py:118-170) with bytes_per_thread=8,
 * threads_per_block=512.  The code table is (code_len[s], code_val[s]) for the
 * 256 byte symbols plus the end-of-stream pseudo-symbol (eof_len, eof_val).
 * Outputs: `encoded` (capacity cap_bytes), `gaps_packed` (5 bits per thread,
 * MSB-first, 320 bytes per block, capacity cap_gap_bytes), `positions`
 * (capacity cap_positions).  As in the reference, `positions` can come out one
 * entry short of n_blocks+1 when the last code crosses a block boundary and
 * ends byte-aligned.
 */
int df11o_encode(const uint8_t *data, int64_t n, const uint8_t *code_len, const uint32_t *code_val,
                 int eof_len, uint32_t eof_val,
                 uint8_t *encoded, int64_t cap_bytes, int64_t *n_bytes_out,
                 uint8_t *gaps_packed, int64_t cap_gap_bytes, int64_t *n_gap_bytes_out,
                 uint32_t *positions, int64_t cap_positions, int64_t *n_positions_out)
{
    const int64_t chunk_bits = 8 * BYTES_PER_THREAD;
    const int64_t block_bits = chunk_bits * N_THREADS;
    int64_t n_enc = 0, n_gaps = 0, n_pos = 0;
    int64_t cap_gaps = cap_gap_bytes * 8 / 5;
    uint8_t *gap_vals = (uint8_t *)malloc((size_t)(cap_gaps > 0 ? cap_gaps : 1));
    uint64_t buffer = 0;
    int size = 0;
    int64_t total_size = 0, element_count = 0;
    int rc = DF11O_OK;

    for (int64_t i = 0; i < n; ++i) {
        uint8_t s = data[i];
        if (total_size / chunk_bits + 1 > n_gaps) {
            if (n_gaps >= cap_gaps) { rc = DF11O_ERR_CAPACITY; goto done; }
            gap_vals[n_gaps++] = (uint8_t)(total_size - total_size / chunk_bits * chunk_bits);
        }
        if (total_size / block_bits + 1 > n_pos) {
            if (n_pos >= cap_positions) { rc = DF11O_ERR_CAPACITY; goto done; }
            positions[n_pos++] = (uint32_t)element_count;
        }
        int b = code_len[s];
        if (b == 0) { rc = DF11O_ERR_ARG; goto done; }
        buffer = (buffer << b) + code_val[s];
        size += b;
        total_size += b;
        element_count += 1;
        while (size >= 8) {
            uint8_t byte = (uint8_t)(buffer >> (size - 8));
            if (n_enc >= cap_bytes) { rc = DF11O_ERR_CAPACITY; goto done; }
            encoded[n_enc++] = byte;
            buffer -= (uint64_t)byte << (size - 8);
            size -= 8;
        }
    }
    if (size > 0) {
        if (total_size / chunk_bits + 1 > n_gaps) {
            if (n_gaps >= cap_gaps) { rc = DF11O_ERR_CAPACITY; goto done; }
            gap_vals[n_gaps++] = (uint8_t)(total_size - total_size / chunk_bits * chunk_bits);
        }
        if (total_size / block_bits + 1 > n_pos) {
            if (n_pos >= cap_positions) { rc = DF11O_ERR_CAPACITY; goto done; }
            positions[n_pos++] = (uint32_t)element_count;
        }
        buffer = (buffer << eof_len) + eof_val;
        size += eof_len;
        uint8_t byte = size >= 8 ? (uint8_t)(buffer >> (size - 8)) : (uint8_t)(buffer << (8 - size));
        if (n_enc >= cap_bytes) { rc = DF11O_ERR_CAPACITY; goto done; }
        encoded[n_enc++] = byte;
    }
    if (n_pos >= cap_positions) { rc = DF11O_ERR_CAPACITY; goto done; }
    positions[n_pos++] = (uint32_t)n;

    {
        int64_t n_blocks = (n_enc + BLOCK_BYTES - 1) / BLOCK_BYTES;
        int64_t n_threads = n_blocks * N_THREADS;
        int64_t gap_bytes = n_threads * 5 / 8;
        if (gap_bytes > cap_gap_bytes || n_gaps > n_threads) { rc = DF11O_ERR_CAPACITY; goto done; }
        memset(gaps_packed, 0, (size_t)gap_bytes);
        /* '05b' per value, concatenated, np.packbits: bit k of the string goes
         * to bit 7-(k%8) of byte k/8. */
        for (int64_t t = 0; t < n_gaps; ++t) {
            for (int k = 0; k < 5; ++k) {
                int bit = (gap_vals[t] >> (4 - k)) & 1;
                int64_t pos = t * 5 + k;
                gaps_packed[pos >> 3] |= (uint8_t)(bit << (7 - (pos & 7)));
            }
        }
        *n_gap_bytes_out = gap_bytes;
    }
    *n_bytes_out = n_enc;
    *n_positions_out = n_pos;
done:
    free(gap_vals);
    return rc;
}
