// Per-chunk decode logic shared by the gfx950 kernels and by a host build used
// for bounds-checked emulation in tests.  Everything here is a pure function of
// its arguments; memory is reached only through the pointers passed in, so the
// same code runs against LDS on the device and against plain arrays on the host.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define DF11_HD __host__ __device__ __forceinline__
#else
#define DF11_HD inline
#endif

namespace df11 {

constexpr int kChunkBytes = 8;        // bytes of bitstream owned by one thread
constexpr int kThreads = 512;         // threads (chunks) per bitstream block
constexpr int kBlockBytes = kChunkBytes * kThreads;
constexpr int kGapBytesPerBlock = kThreads * 5 / 8;
constexpr int kMaxElemsPerBlock = kBlockBytes * 8;   // one-bit codes

// Width of the direct-indexed tables: one lookup resolves every code that
// ends inside the next kK bits of the stream.
constexpr int kK = 12;
constexpr int kTableEntries = 1 << kK;

// Derived table blob (built once per tensor from the byte LUTs):
//   dec  u32[4096]  up to three symbols that end inside the 12-bit window:
//                   sym0 | sym1<<8 | sym2<<16 | bits<<24 | count<<28 ; 0 = first code longer than 12 bits
//   cntf u8[4096]   all codes that end inside the window: count<<4 | bits ; 0 = as above
//   cntt u8[4096]   index (1<<r)|v, v = the next r bits (r < 12): how many codes start inside those r bits
constexpr int kDecOffset = 0;
constexpr int kCntFullOffset = kTableEntries * 4;
constexpr int kCntTailOffset = kCntFullOffset + kTableEntries;
constexpr int kTablesBytes = kCntTailOffset + kTableEntries;

// Byte LUT rows a pointer entry can name: values 255..240 name rows 1..16.
constexpr int kMaxDecodeRows = 17;

struct Luts {
  const uint8_t* rows;   // n_rows decode rows of 256 bytes, then the length row
  int n_rows;            // decode rows present (root included), <= kMaxDecodeRows
};

// Hierarchical lookup of the code at the top of `window`.  A value >= 240 on
// the first three levels names row 256 - value when that row exists.  A symbol
// whose recorded length is 0 can only be reached through padding bits; it is
// given length 1 so that every caller makes progress.
DF11_HD void walk(const Luts& l, uint64_t window, uint32_t& sym, uint32_t& len) {
  uint32_t d = l.rows[window >> 56];
#pragma unroll
  for (int level = 1; level <= 3; ++level) {
    const uint32_t row = 256u - d;
    if (d < 240u || row >= (uint32_t)l.n_rows) break;
    d = l.rows[row * 256u + (uint32_t)((window >> (56 - 8 * level)) & 0xffu)];
  }
  sym = d;
  const uint32_t n = l.rows[(uint32_t)l.n_rows * 256u + d];
  len = n ? n : 1u;
}

// ---- table construction (one entry per call) --------------------------------

DF11_HD uint32_t make_dec_entry(const Luts& l, uint32_t idx) {
  const uint64_t window = (uint64_t)idx << (64 - kK);
  uint32_t pos = 0, k = 0, syms = 0;
  while (k < 3) {
    uint32_t s, n;
    walk(l, window << pos, s, n);
    if (pos + n > (uint32_t)kK) break;
    syms |= s << (8 * k);
    pos += n;
    ++k;
  }
  return k ? (syms | (pos << 24) | (k << 28)) : 0u;
}

DF11_HD uint8_t make_cnt_full_entry(const Luts& l, uint32_t idx) {
  const uint64_t window = (uint64_t)idx << (64 - kK);
  uint32_t pos = 0, k = 0;
  for (;;) {
    uint32_t s, n;
    walk(l, window << pos, s, n);
    if (pos + n > (uint32_t)kK) break;
    pos += n;
    ++k;
    if (pos == (uint32_t)kK) break;
  }
  return (uint8_t)((k << 4) | pos);   // k <= 12, pos <= 12
}

DF11_HD uint8_t make_cnt_tail_entry(const Luts& l, uint32_t idx) {
  if (idx == 0) return 0;
  int r = 31 - __builtin_clz(idx);               // known bits
  if (r == 0) return 0;
  const uint32_t v = idx - (1u << r);
  const uint64_t window = (uint64_t)v << (64 - r);
  uint32_t pos = 0, k = 0;
  while (pos < (uint32_t)r) {
    uint32_t s, n;
    walk(l, window << pos, s, n);
    pos += n;
    ++k;
  }
  return (uint8_t)k;
}

// ---- per-chunk passes ---------------------------------------------------------

struct Tables {
  const uint32_t* dec;
  const uint8_t* cntf;
  const uint8_t* cntt;
};

// Number of codes that start inside the 64-bit chunk {hi,lo}; `next` holds the
// 32 stream bits after the chunk, `gap` the bit offset of the first code start.
DF11_HD uint32_t count_chunk(const Tables& t, const Luts& l, uint32_t hi, uint32_t lo,
                             uint32_t next, uint32_t gap) {
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  uint32_t c = gap, n = 0;
  while (c < 32u) {
    const uint32_t e = t.cntf[(uint32_t)(w >> (64 - kK))];
    uint32_t nb;
    if (e) {
      n += e >> 4;
      nb = e & 15u;
    } else {
      uint32_t s;
      walk(l, w, s, nb);
      n += 1;
    }
    w <<= nb;
    c += nb;
  }
  w |= (uint64_t)next << (c - 32u);
  while (c < 64u) {
    const uint32_t r = 64u - c;
    if (r < (uint32_t)kK) {
      n += t.cntt[(1u << r) | (uint32_t)(w >> (64u - r))];
      break;
    }
    const uint32_t e = t.cntf[(uint32_t)(w >> (64 - kK))];
    uint32_t nb;
    if (e) {
      n += e >> 4;
      nb = e & 15u;
    } else {
      uint32_t s;
      walk(l, w, s, nb);
      n += 1;
    }
    w <<= nb;
    c += nb;
  }
  return n;
}

// Decode the first `remaining` codes of the chunk and write their symbols
// (exponent bytes) to stage[0..remaining).
DF11_HD void emit_chunk(const Tables& t, const Luts& l, uint32_t hi, uint32_t lo, uint32_t next,
                        uint32_t gap, uint32_t remaining, uint8_t* stage) {
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  uint32_t c = gap;
  bool refilled = false;
  while (remaining) {
    if (!refilled && c >= 32u) {
      w |= (uint64_t)next << (c - 32u);
      refilled = true;
    }
    const uint32_t e = t.dec[(uint32_t)(w >> (64 - kK))];
    uint32_t nb;
    if (e) {
      const uint32_t k = e >> 28;
      nb = (e >> 24) & 15u;
      stage[0] = (uint8_t)e;
      if (k > 1u && remaining > 1u) stage[1] = (uint8_t)(e >> 8);
      if (k > 2u && remaining > 2u) stage[2] = (uint8_t)(e >> 16);
      const uint32_t take = k < remaining ? k : remaining;
      stage += take;
      remaining -= take;
    } else {
      uint32_t s;
      walk(l, w, s, nb);
      stage[0] = (uint8_t)s;
      stage += 1;
      remaining -= 1;
    }
    w <<= nb;
    c += nb;
  }
}

// BF16 word from exponent byte and sign|mantissa byte.
DF11_HD uint16_t merge(uint32_t exponent, uint32_t sm) {
  return (uint16_t)(((sm & 0x80u) << 8) | (exponent << 7) | (sm & 0x7fu));
}

// 5-bit gap of chunk `gid` from the MSB-first packed array.
DF11_HD uint32_t gap_of(const uint8_t* gaps, int64_t gid, int64_t n_gap_bytes) {
  const int64_t bit = gid * 5;
  const int64_t byte = bit >> 3;
  const uint32_t b0 = gaps[byte];
  const uint32_t b1 = byte + 1 < n_gap_bytes ? gaps[byte + 1] : 0u;
  return (((b0 << 8) | b1) >> (11 - (int)(bit & 7))) & 31u;
}

// The 8-byte chunk of thread `gid` and the 4 bytes after it, as big-endian
// words; bytes at or beyond n_bytes read as zero.  `aligned`: codes is 8-byte
// aligned, so the chunk can be fetched as one 8-byte and one 4-byte load.
struct Chunk {
  uint32_t hi, lo, next;
};

struct alignas(8) U32x2 {
  uint32_t x, y;
};
struct alignas(16) U32x4 {
  uint32_t x, y, z, w;
};

// Aligned wide access to byte buffers without type punning.
template <class T>
DF11_HD T load_as(const void* p) {
  T v;
  __builtin_memcpy(&v, __builtin_assume_aligned(p, alignof(T)), sizeof(T));
  return v;
}
template <class T>
DF11_HD void store_as(void* p, const T& v) {
  __builtin_memcpy(__builtin_assume_aligned(p, alignof(T)), &v, sizeof(T));
}

DF11_HD Chunk fetch_chunk(const uint8_t* codes, int64_t n_bytes, int64_t gid, bool aligned) {
  const int64_t off = gid * kChunkBytes;
  uint32_t d0 = 0, d1 = 0, d2 = 0;
  if (aligned && off + 12 <= n_bytes) {
    const U32x2 v = load_as<U32x2>(codes + off);
    d0 = v.x;
    d1 = v.y;
    d2 = load_as<uint32_t>(codes + off + 8);
  } else {
    for (int k = 0; k < 4; ++k) {
      if (off + k < n_bytes) d0 |= (uint32_t)codes[off + k] << (8 * k);
      if (off + 4 + k < n_bytes) d1 |= (uint32_t)codes[off + 4 + k] << (8 * k);
      if (off + 8 + k < n_bytes) d2 |= (uint32_t)codes[off + 8 + k] << (8 * k);
    }
  }
  return Chunk{__builtin_bswap32(d0), __builtin_bswap32(d1), __builtin_bswap32(d2)};
}

// Where a bitstream block lands.  The staging area keeps the output's phase
// modulo 8 elements (staging index i holds output element a0 + i), so that
// 8-byte staging reads pair with 8-byte sign|mantissa loads and 16-byte stores.
struct BlockPlan {
  int64_t a0;       // output index of staging index 0 (multiple of 8)
  uint32_t phase;   // staging index of the block's first element, 0..7
  uint32_t n_out;   // elements this block produces (clamped to n_elements and to the staging capacity)
};

DF11_HD BlockPlan plan_block(int64_t base, uint32_t total, int64_t n_elements, int32_t stage_cap) {
  BlockPlan p;
  p.a0 = base & ~(int64_t)7;
  p.phase = (uint32_t)(base - p.a0);
  int64_t end = base + (int64_t)total;
  if (end > n_elements) end = n_elements;
  int64_t n_out = end > base ? end - base : 0;
  const int64_t room = (int64_t)stage_cap - (int64_t)p.phase;
  if (n_out > room) n_out = room;
  p.n_out = (uint32_t)n_out;
  return p;
}

// How many of its `count` codes a thread with exclusive prefix `excl` decodes.
DF11_HD uint32_t thread_quota(uint32_t excl, uint32_t count, uint32_t n_out) {
  uint32_t my_end = excl + count;
  if (my_end > n_out) my_end = n_out;
  return my_end > excl ? my_end - excl : 0u;
}

DF11_HD uint32_t n_groups_of(const BlockPlan& p) { return (p.phase + p.n_out + 7u) >> 3; }

// bytes 0,1 (or 2,3) of x moved to the low bytes of the two 16-bit halves
DF11_HD uint32_t spread_lo(uint32_t x) { return (x & 0xffu) | ((x & 0xff00u) << 8); }
DF11_HD uint32_t spread_hi(uint32_t x) { return ((x >> 16) & 0xffu) | ((x >> 8) & 0xff0000u); }
DF11_HD uint32_t merge2(uint32_t e, uint32_t m) {   // two BF16 words per 32-bit word
  return ((m & 0x00800080u) << 8) | (e << 7) | (m & 0x007f007fu);
}

// Write output group g of the block: elements a0 + 8g .. a0 + 8g + 7 that
// belong to the block.  `vec_ok`: sign_mantissa is 8-byte and out 16-byte aligned.
DF11_HD void stream_group(uint32_t g, const BlockPlan& p, const uint8_t* stage,
                          const uint8_t* sign_mantissa, uint16_t* out, bool vec_ok) {
  const uint32_t first = p.phase, last = p.phase + p.n_out;
  const uint32_t s0 = g << 3;
  if (vec_ok && s0 >= first && s0 + 8u <= last) {
    const U32x2 e8 = load_as<U32x2>(stage + s0);
    const U32x2 m8 = load_as<U32x2>(sign_mantissa + p.a0 + s0);
    U32x4 o;
    o.x = merge2(spread_lo(e8.x), spread_lo(m8.x));
    o.y = merge2(spread_hi(e8.x), spread_hi(m8.x));
    o.z = merge2(spread_lo(e8.y), spread_lo(m8.y));
    o.w = merge2(spread_hi(e8.y), spread_hi(m8.y));
    store_as<U32x4>(out + p.a0 + s0, o);
  } else {
    const uint32_t lo_i = s0 > first ? s0 : first;
    const uint32_t hi_i = s0 + 8u < last ? s0 + 8u : last;
    for (uint32_t i = lo_i; i < hi_i; ++i) out[p.a0 + i] = merge(stage[i], sign_mantissa[p.a0 + i]);
  }
}

}  // namespace df11
