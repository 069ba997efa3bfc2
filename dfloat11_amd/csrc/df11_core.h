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

// Width of the direct-indexed table: one lookup resolves up to four codes that
// end inside the next kK bits of the stream.
constexpr int kK = 11;
constexpr int kTableEntries = 1 << kK;

// Derived table blob (built once per tensor from the byte LUTs):
//   dec  u32[2048][2]  word 0: the symbols of up to four codes that end inside the
//                      11-bit window, first code in byte 0;
//                      word 1 ("meta"): bits consumed in byte 0, code count in
//                      byte 1; 0 = the first code is longer than 11 bits
//   cntt u8[2048]      index (1<<r)|v, v = the next r bits (r < 11): how many codes
//                      start inside those r bits
constexpr int kDecOffset = 0;
constexpr int kCntTailOffset = kTableEntries * 8;
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

// Is the code at the top of `window` settled by its first `known` bits alone?
// The byte LUTs answer for any 8-bit index, including indices whose low bits
// are not known yet; the answer counts only if it uses no more than the known
// bits AND does not change when the unknown bits do.  The second condition
// rejects slots that merely inherited a neighbour's symbol (the end-of-stream
// code's slots, unused code space): there the symbol found with the unknown
// bits at 0 and at 1 differs, or its length exceeds the known bits.
DF11_HD bool resolve(const Luts& l, uint64_t window, uint32_t known, uint32_t& sym, uint32_t& len) {
  if (known == 0) return false;
  const uint64_t unknown_mask = known >= 64u ? 0ull : (~0ull >> known);
  uint32_t s0, n0, s1, n1;
  walk(l, window & ~unknown_mask, s0, n0);
  walk(l, window | unknown_mask, s1, n1);
  sym = s0;
  len = n0;
  return n0 <= known && s0 == s1 && n0 == n1;
}

DF11_HD void make_dec_entry(const Luts& l, uint32_t idx, uint32_t& syms, uint32_t& meta) {
  const uint64_t window = (uint64_t)idx << (64 - kK);
  uint32_t pos = 0, k = 0;
  syms = 0;
  while (k < 4) {
    uint32_t s, n;
    if (!resolve(l, window << pos, (uint32_t)kK - pos, s, n)) break;
    syms |= s << (8 * k);
    pos += n;
    ++k;
  }
  meta = k ? (pos | (k << 8)) : 0u;
  if (!k) syms = 0;
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
    ++k;                                          // a code starts at pos
    if (!resolve(l, window << pos, (uint32_t)r - pos, s, n)) break;   // and runs past the known bits
    pos += n;
  }
  return (uint8_t)k;
}

// ---- per-chunk passes ---------------------------------------------------------

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

struct Tables {
  const uint8_t* dec;     // u32[2048][2], 8-byte aligned
  const uint8_t* cntt;    // u8[2048]
};

// Unaligned 32-/16-bit stores (LDS supports them on gfx950; one instruction each).
DF11_HD void store32(uint8_t* p, uint32_t v) { __builtin_memcpy(p, &v, 4); }
DF11_HD void store16(uint8_t* p, uint32_t v) {
  const uint16_t h = (uint16_t)v;
  __builtin_memcpy(p, &h, 2);
}

// Keeps a rarely taken branch a branch: without it the compiler turns the body
// into unconditional selects that every loop iteration pays for.
#if defined(__HIP_DEVICE_COMPILE__)
#define DF11_KEEP_BRANCH() asm volatile("" ::: "memory")
#else
#define DF11_KEEP_BRANCH() ((void)0)
#endif

// The window with the 32 look-ahead bits appended below its 64 - c valid bits.
DF11_HD uint64_t with_next(uint64_t w, uint32_t next, uint32_t c) {
  if (c == 0) return w;
  return w | (c >= 32u ? (uint64_t)next << (c - 32u) : (uint64_t)next >> (32u - c));
}

// Byte offset of the table entry for the top kK bits of the window.
DF11_HD uint32_t dec_offset(uint64_t w) { return ((uint32_t)(w >> 32) >> (32 - kK - 3)) & (uint32_t)((kTableEntries - 1) * 8); }

// Number of codes that start inside the 64-bit chunk {hi,lo}; `next` holds the
// 32 stream bits after the chunk, `gap` the bit offset of the first code start.
// Lookups stay inside the chunk (c <= 64 - kK), so the look-ahead is only needed
// for codes longer than the table width; the last few bits are settled by one
// lookup in the tail table.
DF11_HD uint32_t count_chunk(const Tables& t, const Luts& l, uint32_t hi, uint32_t lo,
                             uint32_t next, uint32_t gap) {
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  uint32_t cn = gap;                    // byte 0: bits consumed; bits 8 and up: codes counted
  while ((cn & 0xffu) <= 64u - (uint32_t)kK) {
    uint32_t meta = load_as<uint32_t>(t.dec + dec_offset(w) + 4u);
    if (meta == 0u) {
      uint32_t s, n;
      walk(l, with_next(w, next, cn & 0xffu), s, n);
      meta = n | 0x100u;
      DF11_KEEP_BRANCH();
    }
    w <<= (meta & 63u);
    cn += meta;
  }
  const uint32_t c = cn & 0xffu;
  uint32_t n = cn >> 8;
  if (c < 64u) n += t.cntt[(1u << (64u - c)) | (uint32_t)(w >> c)];
  return n;
}

// Decode the first `remaining` codes of the chunk and write their symbols
// (exponent bytes) to p[0..remaining).  While four or more bytes remain the
// four symbol bytes of a lookup are stored at once: bytes past the codes it
// resolved are overwritten by the next store.  The last one to three symbols
// are gathered in a register and stored exactly, so nothing is ever written at
// or beyond p + remaining.
DF11_HD void emit_chunk(const Tables& t, const Luts& l, uint32_t hi, uint32_t lo, uint32_t next,
                        uint32_t gap, uint32_t remaining, uint8_t* p) {
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  uint32_t c = gap;                     // bit 7 is set once the look-ahead has been appended
  uint32_t rem = remaining;
  while (rem >= 4u) {
    if (c - 32u < 96u) {                // 32 <= c < 128: room for the look-ahead, not yet appended
      w |= (uint64_t)next << (c - 32u);
      c += 128u;
      DF11_KEEP_BRANCH();
    }
    const U32x2 e = load_as<U32x2>(t.dec + dec_offset(w));
    uint32_t syms = e.x, meta = e.y;
    if (meta == 0u) {
      uint32_t n;
      walk(l, w, syms, n);              // at least 32 valid bits: c < 32, or already appended
      meta = n | 0x100u;
      DF11_KEEP_BRANCH();
    }
    store32(p, syms);
    const uint32_t k = meta >> 8;
    p += k;
    rem -= k;
    w <<= (meta & 63u);
    c += meta & 0xffu;
  }
  if (rem) {
    uint32_t acc = 0, got = 0;          // got: bits gathered, 8 per symbol
    while (got < 8u * rem) {
      if (c - 32u < 96u) {
        w |= (uint64_t)next << (c - 32u);
        c += 128u;
      }
      const U32x2 e = load_as<U32x2>(t.dec + dec_offset(w));
      uint32_t syms = e.x, meta = e.y;
      if (meta == 0u) {
        uint32_t n;
        walk(l, w, syms, n);
        meta = n | 0x100u;
      }
      acc |= syms << got;
      got += 8u * (meta >> 8);
      w <<= (meta & 63u);
      c += meta & 0xffu;
    }
    if (rem & 2u) store16(p, acc);
    if (rem & 1u) p[rem & 2u] = (uint8_t)(acc >> (8u * (rem & 2u)));
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
// modulo 16 elements (staging index i holds output element a0 + i), so that
// 16-byte staging reads pair with 16-byte sign|mantissa loads and 32 bytes of
// BF16 stores.
struct BlockPlan {
  int64_t a0;       // output index of staging index 0 (multiple of 16)
  uint32_t phase;   // staging index of the block's first element, 0..15
  uint32_t n_out;   // elements this block produces (clamped to n_elements and to the staging capacity)
};

constexpr int kGroup = 16;   // elements per lane per write-out step

DF11_HD BlockPlan plan_block(int64_t base, uint32_t total, int64_t n_elements, int32_t stage_cap) {
  BlockPlan p;
  p.a0 = base & ~(int64_t)(kGroup - 1);
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

DF11_HD uint32_t n_groups_of(const BlockPlan& p) {
  return (p.phase + p.n_out + (uint32_t)kGroup - 1u) / (uint32_t)kGroup;
}

// Four BF16 words from four exponent bytes E and four sign|mantissa bytes S:
// high bytes (S & 0x80) | (E >> 1), low bytes (E << 7) | (S & 0x7f), interleaved.
DF11_HD void merge4(uint32_t E, uint32_t S, uint32_t& out01, uint32_t& out23) {
  const uint32_t hi = (S & 0x80808080u) | ((E >> 1) & 0x7f7f7f7fu);
  const uint32_t lo = ((E << 7) & 0x80808080u) | (S & 0x7f7f7f7fu);
#if defined(__HIP_DEVICE_COMPILE__)
  out01 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);   // lo0 hi0 lo1 hi1
  out23 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);   // lo2 hi2 lo3 hi3
#else
  out01 = (lo & 0xffu) | ((hi & 0xffu) << 8) | ((lo & 0xff00u) << 8) | ((hi & 0xff00u) << 16);
  out23 = ((lo >> 16) & 0xffu) | ((hi >> 8) & 0xff00u) | ((lo >> 8) & 0xff0000u) | (hi & 0xff000000u);
#endif
}

// True when group g of the block can take the 16-wide path.
DF11_HD bool group_is_full(uint32_t g, const BlockPlan& p) {
  const uint32_t s0 = g * (uint32_t)kGroup;
  return s0 >= p.phase && s0 + (uint32_t)kGroup <= p.phase + p.n_out;
}

// 16-wide path: `m` holds the 16 sign|mantissa bytes of the group (loaded by the
// caller, possibly long before), staging bytes come from `stage`.
DF11_HD void stream_group_full(uint32_t g, const BlockPlan& p, const uint8_t* stage, const U32x4& m,
                               uint16_t* out) {
  const uint32_t s0 = g * (uint32_t)kGroup;
  const U32x4 e = load_as<U32x4>(stage + s0);
  U32x4 o0, o1;
  merge4(e.x, m.x, o0.x, o0.y);
  merge4(e.y, m.y, o0.z, o0.w);
  merge4(e.z, m.z, o1.x, o1.y);
  merge4(e.w, m.w, o1.z, o1.w);
  store_as<U32x4>(out + p.a0 + s0, o0);
  store_as<U32x4>(out + p.a0 + s0 + 8, o1);
}

// Element-wise path for the ragged ends of a block (and for unaligned buffers).
DF11_HD void stream_group_ragged(uint32_t g, const BlockPlan& p, const uint8_t* stage,
                                 const uint8_t* sign_mantissa, uint16_t* out) {
  const uint32_t first = p.phase, last = p.phase + p.n_out;
  const uint32_t s0 = g * (uint32_t)kGroup;
  const uint32_t lo_i = s0 > first ? s0 : first;
  const uint32_t hi_i = s0 + (uint32_t)kGroup < last ? s0 + (uint32_t)kGroup : last;
  for (uint32_t i = lo_i; i < hi_i; ++i) out[p.a0 + i] = merge(stage[i], sign_mantissa[p.a0 + i]);
}

}  // namespace df11
