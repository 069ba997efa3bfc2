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

// Pointers into workgroup memory (LDS) carry their address space on the device,
// so that accesses compile to LDS instructions with constant parts of the address
// in the instruction's offset field; on the host they are plain pointers.
#if defined(__HIP_DEVICE_COMPILE__)
#define DF11_LDS __attribute__((address_space(3)))
#else
#define DF11_LDS
#endif

namespace df11 {

typedef DF11_LDS uint8_t* LdsBytes;
typedef const DF11_LDS uint8_t* ConstLdsBytes;

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
//                      byte 1.  When the first code is longer than 11 bits, bit 31
//                      of word 1 is set and the two words say where the code's
//                      hierarchical lookup starts (start_of_unsettled): word 0 the
//                      byte offset of a fused row, bits 0-4 of word 1 the position
//                      of the code byte that indexes it
//   cntt u8[2048]      index (1<<r)|v, v = the next r bits (r < 11): how many codes
//                      start inside those r bits
//   rows u16[n_rows][256]  the byte LUT rows fused with the length row: bits 0-7 the
//                      row's byte d, bits 8-14 the recorded code length of symbol d
//                      (1 where it is 0), bit 15 set if d names a row that exists
//                      (d >= 240 and 256 - d < n_rows): a pointer on levels 0-2
constexpr int kDecOffset = 0;
constexpr int kCntTailOffset = kTableEntries * 8;
constexpr int kRowsOffset = kCntTailOffset + kTableEntries;

// Byte LUT rows a pointer entry can name: values 255..240 name rows 1..16.
constexpr int kMaxDecodeRows = 17;
constexpr int kRowBytes = 256 * 2;
constexpr int kTablesBytes = kRowsOffset + kMaxDecodeRows * kRowBytes;   // the blob with every row present
// Bytes of the blob a decode needs when the stream has n_rows decode rows.
DF11_HD int tables_bytes(int n_rows) { return kRowsOffset + n_rows * kRowBytes; }

struct Luts {
  const uint8_t* rows;   // n_rows decode rows of 256 bytes, then the length row
  int n_rows;            // decode rows present (root included), <= kMaxDecodeRows
};

// Fused entry of byte `byte` of row `row`: what a hierarchical lookup needs to know
// about that slot, in one 16-bit read.  A symbol whose recorded length is 0 can
// only be reached through padding bits; it is given length 1 so that every
// caller makes progress.
constexpr uint32_t kRowPointer = 0x8000u;
DF11_HD uint16_t make_row_entry(const Luts& l, uint32_t row, uint32_t byte) {
  const uint32_t d = l.rows[row * 256u + byte];
  uint32_t n = l.rows[(uint32_t)l.n_rows * 256u + d];
  if (n > 127u) n = 127u;                      // a valid length is at most 32; keeps bit 15 for the flag
  const bool names_row = d >= 240u && 256u - d < (uint32_t)l.n_rows;
  return (uint16_t)(d | ((n ? n : 1u) << 8) | (names_row ? kRowPointer : 0u));
}

// ---- table construction (one entry per call) --------------------------------

// Is the code at the top of `window` settled by its first `known` bits alone?
// If so, returns its symbol and length.  The bits of `window` below the known
// ones must be zero.
//
// The byte LUTs answer for any 8-bit index, including indices whose low bits
// are not known yet and slots that no code owns (the end-of-stream code's
// slots, unused code space), which hold whatever the builder of the LUTs filled
// them with.  The rule below is independent of that filling.  Whole known bytes
// index slots that a code or a pointer owns (the known bits start a code of the
// stream).  Where the known bits end inside a byte, the code is settled only if
// every slot that the unknown bits can select holds the same symbol, and that
// symbol's recorded length belongs to this level (8*level+1 .. 8*level+8) and
// fits into the known bits: if the known bits were only the beginning of a
// longer code, that code's own slots (or the pointer towards it) would lie
// among the selected ones and either differ from the rest or, when all of them
// are equal, be an entry longer than the known bits.
DF11_HD bool resolve(const Luts& l, uint64_t window, uint32_t known, uint32_t& sym, uint32_t& len) {
  uint32_t row = 0;
  for (uint32_t level = 0; level <= 3u; ++level) {
    if (known <= 8u * level) return false;                   // nothing known of this byte
    const uint32_t kb = known - 8u * level;                  // known bits of this byte, 8 = all
    const uint32_t lo = (uint32_t)(window >> (56u - 8u * level)) & 0xffu;
    const uint32_t d = l.rows[row * 256u + lo];
    if (kb < 8u) {
      const uint32_t hi = lo | (0xffu >> kb);
      if (l.rows[row * 256u + hi] != d) return false;          // the usual way out for an unsettled code
      for (uint32_t j = lo + 1u; j < hi; ++j)
        if (l.rows[row * 256u + j] != d) return false;
    }
    const uint32_t next_row = 256u - d;
    if (level < 3u && d >= 240u && next_row < (uint32_t)l.n_rows) {   // a pointer
      if (kb < 8u) return false;                             // the code continues past the known bits
      row = next_row;
      continue;
    }
    const uint32_t n = l.rows[(uint32_t)l.n_rows * 256u + d];
    if (n <= 8u * level || n > 8u * level + 8u) return false;   // not an entry of this level: filling
    sym = d;
    len = n;
    return n <= known;
  }
  return false;
}

// Where the hierarchical lookup may start for an 11-bit window `idx` that settles
// no code (so every code word that begins with these bits is longer than 11
// bits): the byte offset of a fused row, and the position (24, 16, 8 or 0) in the
// code's first 32 bits of the byte that indexes that row, marked with kUnsettled.
// From the root the lookup follows a pointer per level; a level
// can be skipped ahead of time when every slot the unknown bits can select
// either holds one and the same pointer or is a symbol whose recorded length does
// not belong to that level (8*level+1 .. 8*level+8): such a slot is filling that
// no code word owns, so every code word with these leading bits goes through
// that pointer.  Codes that pad a stem with fixed bits (the long codes given to
// exponents >= 240) then need one row read instead of three.
constexpr uint32_t kUnsettled = 0x80000000u;
DF11_HD void start_of_unsettled(const Luts& l, uint32_t idx, uint32_t& row_offset, uint32_t& at) {
  uint32_t row = 0, level = 0;
  while (level < 3u) {
    const int known = kK - 8 * (int)level;                       // bits of this level's byte that idx fixes
    const uint32_t kb = known >= 8 ? 8u : known > 0 ? (uint32_t)known : 0u;
    const uint32_t lo = kb ? ((idx >> (kK - 8 * (int)level - (int)kb)) & ((1u << kb) - 1u)) << (8u - kb) : 0u;
    const uint32_t n = 1u << (8u - kb);
    uint32_t pointer = 0;                                        // the one pointer seen, 0 = none yet
    bool skip = true;
    for (uint32_t j = lo; j < lo + n; ++j) {
      const uint32_t d = l.rows[row * 256u + j];
      if (d >= 240u && 256u - d < (uint32_t)l.n_rows) {
        if (pointer && pointer != d) skip = false;
        pointer = d;
      } else {
        const uint32_t len = l.rows[(uint32_t)l.n_rows * 256u + d];
        if (len > 8u * level && len <= 8u * level + 8u) skip = false;   // may be a code word's own slot
      }
    }
    if (!skip || !pointer) break;
    row = 256u - pointer;
    ++level;
  }
  row_offset = row * (uint32_t)kRowBytes;
  at = kUnsettled | (24u - 8u * level);
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
  meta = pos | (k << 8);
  if (!k) start_of_unsettled(l, idx, syms, meta);
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

// The same for workgroup memory; p is aligned to alignof(T).
#if defined(__HIP_DEVICE_COMPILE__)
#define DF11_LDS_ALIGNED(p, n) __builtin_assume((reinterpret_cast<uintptr_t>(p) & ((n) - 1)) == 0)
#else
#define DF11_LDS_ALIGNED(p, n) ((void)0)
#endif
template <class T>
DF11_HD T lds_load(ConstLdsBytes p) {
  DF11_LDS_ALIGNED(p, alignof(T));
  T v;
  __builtin_memcpy(&v, p, sizeof(T));
  return v;
}
template <class T>
DF11_HD void lds_store(LdsBytes p, const T& v) {
  DF11_LDS_ALIGNED(p, alignof(T));
  __builtin_memcpy(p, &v, sizeof(T));
}

// The fused rows as the decode reads them (LDS on the device).
struct Rows {
  ConstLdsBytes e;   // u16[n_rows][256], 2-byte aligned
};

// One fused entry, zero-extended.  The compiler is not told that the upper half is
// zero: it would otherwise test the pointer flag on the 16-bit value and extend
// that again for every later use.
DF11_HD uint32_t row_entry_at(const Rows& r, uint32_t byte_offset) {
  uint32_t e = lds_load<uint16_t>(r.e + byte_offset);
#if defined(__HIP_DEVICE_COMPILE__)
  asm("" : "+v"(e));
  __builtin_assume(e < 65536u);
#endif
  return e;
}

// Hierarchical lookup of the code whose first 32 bits are `top` (first bit in
// bit 31), started in the row at byte offset `row_offset` of the fused rows,
// which the code's byte at bits [at & 31, +8) of `top` indexes (24 = first
// byte of the code, 0 = fourth).  A value >= 240 on the first three
// levels names row 256 - value when that row exists; on the fourth level it is
// a symbol.  Row offset 0 with at = 24 is the lookup from the root as the
// reference does it; the table entry of an 11-bit window that settles no code
// holds a start further down where that is safe (start_of_unsettled).
// `at` is kUnsettled | position, as the table holds it.  Returns the fused entry
// of the symbol.
DF11_HD uint32_t byte_at(uint32_t word, uint32_t shift) {   // bits [shift & 31, +8) of word
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_ubfe(word, shift, 8u);           // the instruction reads five bits of the shift
#else
  return (word >> (shift & 31u)) & 0xffu;
#endif
}

DF11_HD uint32_t walk_from(const Rows& r, uint32_t row_offset, uint32_t at, uint32_t top) {
  uint32_t e = row_entry_at(r, row_offset + byte_at(top, at) * 2u);
  while (at != kUnsettled && e >= kRowPointer) {
    at -= 8u;
    e = row_entry_at(r, ((256u - (e & 0xffu)) * 256u + byte_at(top, at)) * 2u);
  }
  return e;
}
DF11_HD uint32_t entry_symbol(uint32_t e) { return e & 0xffu; }
DF11_HD uint32_t entry_length(uint32_t e) { return (e >> 8) & 0x7fu; }
// One code of entry_length bits, as the second word of a table entry.
DF11_HD uint32_t entry_meta(uint32_t e) { return entry_length(e) | 0x100u; }


struct Tables {
  ConstLdsBytes dec;     // u32[2048][2], 8-byte aligned
  ConstLdsBytes cntt;    // u8[2048]
};

// Keeps a rarely taken branch a branch: without it the compiler turns the body
// into unconditional selects that every loop iteration pays for.
#if defined(__HIP_DEVICE_COMPILE__)
#define DF11_KEEP_BRANCH() asm volatile("" ::: "memory")
#else
#define DF11_KEEP_BRANCH() ((void)0)
#endif

// The next 32 stream bits at the top of window `w`, of which the 64 - c topmost
// bits are valid chunk bits and the rest zero (c < 64); `next31` holds the 32 bits
// that follow the chunk, shifted left by 31 (look_ahead): moved down by 63 - c
// they line up with the window's first invalid bit.
DF11_HD uint64_t look_ahead(uint32_t next) { return (uint64_t)next << 31; }
// The window with the look-ahead bits appended below its 64 - c valid bits.
DF11_HD uint64_t with_next(uint64_t w, uint64_t next31, uint32_t c) { return w | (next31 >> (63u - c)); }
DF11_HD uint32_t top_bits(uint64_t w, uint64_t next31, uint32_t c) { return (uint32_t)(with_next(w, next31, c) >> 32); }

// Byte offset of the table entry for the top kK bits of the window.
DF11_HD uint32_t dec_offset(uint64_t w) { return ((uint32_t)(w >> 32) >> (32 - kK - 3)) & (uint32_t)((kTableEntries - 1) * 8); }

// Number of codes that start inside the 64-bit chunk {hi,lo}; `next` holds the
// 32 stream bits after the chunk, `gap` the bit offset of the first code start.
// Lookups stay inside the chunk (c <= 64 - kK), so the look-ahead is only needed
// for codes longer than the table width; the last few bits are settled by one
// lookup in the tail table.
DF11_HD uint32_t count_chunk(const Tables& t, const Rows& l, uint32_t hi, uint32_t lo,
                             uint32_t next, uint32_t gap) {
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  const uint64_t next31 = look_ahead(next);
  uint32_t cn = gap;                    // byte 0: bits consumed; bits 8 and up: codes counted
  while ((cn & 0xffu) <= 64u - (uint32_t)kK) {
    uint32_t meta = lds_load<uint32_t>(t.dec + dec_offset(w) + 4u);
    if (meta & kUnsettled) {
      meta = entry_meta(walk_from(l, lds_load<uint32_t>(t.dec + dec_offset(w)), meta, top_bits(w, next31, cn & 0xffu)));
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

// Decode the first `remaining` codes of the chunk and OR their symbols (exponent
// bytes) into stage[at .. at + remaining), which must hold zeros (`stage` is 4-byte
// aligned, at >= 4).  Each lookup's symbol bytes go out as two aligned words, as in
// replay_chunk; the last lookup is cut to the codes that remain, so nothing is
// written at or beyond at + remaining except zeros.
DF11_HD void emit_chunk(const Tables& t, const Rows& l, uint32_t hi, uint32_t lo, uint32_t next,
                        uint32_t gap, uint32_t remaining, LdsBytes stage, uint32_t at);

// ---- one decode per chunk, kept in registers -------------------------------------
// The fast path decodes a chunk once.  The lookups of a chunk are few (each
// resolves up to four codes), so their results fit in registers: kMain lookups
// that stay inside the chunk plus kTailSlots for the codes that reach into the
// look-ahead (a tail lookup may hold symbols of the next chunk as well: they are
// the true next symbols of the stream).  Once the lane's output offset is known,
// the symbols are replayed into the staging area with no further table access.
// A chunk that needs more lookups than there are slots reports `overflow` and the bit
// at which the rest of it starts: that rest is counted by count_chunk and, once the
// lane's offset is known, decoded a second time by emit_chunk, so the cost of running
// out of slots grows with the lookups that did not fit.
// How many lookups a chunk needs depends on the code: weight-like streams (2.6 bits
// per code, 3.3 codes per lookup) need seven inside the chunk; codes of six to eight
// bits resolve one per lookup and need up to ten; streams of one- to three-bit
// codes (sparse weights) resolve four per lookup and need up to fourteen (a lookup
// inside the chunk starts at bit 53 or before and consumes at least four bits
// unless a code that does not fit the window follows).  The kernel is compiled for
// several slot counts; slots that no lane of a wavefront uses cost a compare and a
// branch each.  Seven is what fits the 64 registers of eight wavefronts per SIMD.
constexpr int kMainSlotsUsual = 10;        // wide (six wavefronts per SIMD), portable, rows
constexpr int kMainSlotsFew = 7;           // the compilations for eight wavefronts per SIMD
constexpr int kMainSlotsDeep = 8;          // large weight-like streams: a ninth changes nothing there, a tenth costs 1 %
constexpr int kMainSlotsShortCodes = 14;   // deepest
constexpr int kTailSlots = 2;

template <int kMain>
struct ChunkSyms {
  static constexpr int kSlots = kMain + kTailSlots;
  uint32_t syms[kSlots];             // symbol bytes of lookup i, first code in byte 0, unused bytes zero
  uint32_t ends[kSlots - 1];         // symbols of the chunk up to and including lookup i
  uint32_t count;                    // codes that start in the chunk; if `overflow`, those of the main lookups only
  uint32_t resume;                   // bit of the chunk at which the lookups after the main ones start
  bool overflow;                     // ran out of slots: the codes from bit `resume` on are not in syms (the
                                     // tail slots are empty then) and not in count
};

// kResume: the caller continues an overflowing chunk from `resume`; without it the caller
// decodes such a chunk again from its start and needs nothing but the flag.
template <int kMain, bool kResume>
DF11_HD ChunkSyms<kMain> decode_chunk_regs(const Tables& t, const Rows& l, uint32_t hi, uint32_t lo,
                                           uint32_t next, uint32_t gap) {
  constexpr int kSlots = ChunkSyms<kMain>::kSlots;
  ChunkSyms<kMain> r;
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  const uint64_t next31 = look_ahead(next);
  uint32_t c = gap, n = 0;
#pragma unroll
  for (int i = 0; i < kMain; ++i) {
    r.syms[i] = 0;
    if (c <= 64u - (uint32_t)kK) {          // the lookup stays inside the chunk
      const U32x2 e = lds_load<U32x2>(t.dec + dec_offset(w));
      uint32_t syms = e.x, meta = e.y;
      if (meta & kUnsettled) {
        const uint32_t long_code = walk_from(l, syms, meta, top_bits(w, next31, c));
        syms = entry_symbol(long_code);
        meta = entry_meta(long_code);
        DF11_KEEP_BRANCH();
      }
      r.syms[i] = syms;
      n += (meta >> 8) & 0xffu;
      w <<= (meta & 63u);
      c += meta & 0xffu;
    }
    r.ends[i] = n;                            // also for a lane that skipped the lookup: later ones start here
  }
  r.overflow = c <= 64u - (uint32_t)kK;
  r.resume = c;
  const uint32_t n_main = n;
  uint32_t todo = 0;                          // codes that still start before the chunk ends
  if (!r.overflow && c < 64u) {
    todo = t.cntt[(1u << (64u - c)) | (uint32_t)(w >> c)];
    w = with_next(w, next31, c);
  }
#pragma unroll
  for (int i = 0; i < kTailSlots; ++i) {
    r.syms[kMain + i] = 0;
    if (todo) {
      const U32x2 e = lds_load<U32x2>(t.dec + dec_offset(w));
      uint32_t syms = e.x, meta = e.y;
      if (meta & kUnsettled) {
        const uint32_t long_code = walk_from(l, syms, meta, (uint32_t)(w >> 32));
        syms = entry_symbol(long_code);
        meta = entry_meta(long_code);
      }
      r.syms[kMain + i] = syms;
      const uint32_t k = meta >> 8;
      const uint32_t take = k < todo ? k : todo;
      n += take;
      todo -= take;
      w <<= (meta & 63u);
    }
    if (kMain + i < kSlots - 1) r.ends[kMain + i] = n;
  }
  if (todo != 0u) {                           // more tail lookups than slots: leave the whole tail to the caller
    r.overflow = true;
    if (kResume) {
#pragma unroll
      for (int i = 0; i < kTailSlots; ++i) r.syms[kMain + i] = 0;
      n = n_main;
    }
  }
  r.count = n;
  return r;
}

// OR a 32-bit value into the aligned word at p.  On the device this is an LDS
// atomic without return: it costs the same as an aligned store, where a store
// to an address that is not a multiple of four stalls the LDS pipeline for
// dozens of cycles.
DF11_HD void or32_aligned(LdsBytes p, uint32_t v) {
  typedef uint32_t __attribute__((may_alias)) Word;
  DF11_LDS Word* w = reinterpret_cast<DF11_LDS Word*>(p);
#if defined(__HIP_DEVICE_COMPILE__)
  __hip_atomic_fetch_or(w, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#else
  *w |= v;
#endif
}

// The 32-bit word that starts `bytes & 3` bytes into the 8-byte value {hi, lo}.
DF11_HD uint32_t align_bytes(uint32_t hi, uint32_t lo, uint32_t bytes) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_alignbyte(hi, lo, bytes);        // the instruction reads two bits of `bytes`
#else
  return (uint32_t)((((uint64_t)hi << 32) | lo) >> (8u * (bytes & 3u)));
#endif
}

// Is `pred` true in any lane of the wavefront?  (On the host every lane is emulated on
// its own and answers for itself.)
DF11_HD bool any_lane(bool pred) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_ballot_w64(pred) != 0;
#else
  return pred;
#endif
}

// Main slots from this one on are there for the streams that need them: they are skipped
// when no lane of the wavefront holds symbols in them (symbol bytes that are all zero
// change nothing when ORed).  The slots before it, and the tail slots, are in use in
// nearly every wavefront of any stream.
constexpr int kFirstOptionalSlot = 7;

// OR the chunk's symbols into stage[at .. at + r.count), which must hold zeros
// (`stage` is 4-byte aligned, at >= 4).  Each lookup's four symbol bytes go out as
// two aligned words, shifted to their byte position; the unused bytes of a lookup
// are zero and leave their neighbours alone, so no lookup needs trimming and the
// lanes of a wavefront may write the bytes of one word in any order.
// The two words are those at and after (pos - 1) & ~3, so that the shift is
// (-pos) & 3 bytes to the right of {symbols, 0}, which one instruction per word
// does from -pos itself; a lookup that starts on a word boundary ORs zero into the
// word before it.
template <int kMain>
DF11_HD void replay_chunk(const ChunkSyms<kMain>& r, LdsBytes stage, uint32_t at) {
  const uint32_t minus_at = 0u - at;
#pragma unroll
  for (int i = 0; i < ChunkSyms<kMain>::kSlots; ++i) {
    if (i >= kFirstOptionalSlot && i < kMain && !any_lane(r.syms[i] != 0u)) continue;
    // lookup i starts where the lookups before it end
    const uint32_t minus_pos = i == 0 ? minus_at : minus_at - r.ends[i - 1];
    LdsBytes w = stage + (~minus_pos & ~3u);               // (pos - 1) & ~3
    or32_aligned(w, align_bytes(r.syms[i], 0u, minus_pos));
    or32_aligned(w + 4, align_bytes(0u, r.syms[i], minus_pos));
  }
}

DF11_HD void emit_chunk(const Tables& t, const Rows& l, uint32_t hi, uint32_t lo, uint32_t next,
                        uint32_t gap, uint32_t remaining, LdsBytes stage, uint32_t at) {
  uint64_t w = (((uint64_t)hi << 32) | lo) << gap;
  uint32_t c = gap;                     // bit 7 is set once the look-ahead has been appended
  uint32_t rem = remaining;
  uint32_t minus_pos = 0u - at;
  while (rem) {
    if (c - 32u < 96u) {                // 32 <= c < 128: room for the look-ahead, not yet appended
      w |= (uint64_t)next << (c - 32u);
      c += 128u;
      DF11_KEEP_BRANCH();
    }
    const U32x2 e = lds_load<U32x2>(t.dec + dec_offset(w));
    uint32_t syms = e.x, meta = e.y;
    if (meta & kUnsettled) {
      const uint32_t long_code = walk_from(l, syms, meta, (uint32_t)(w >> 32));   // at least 32 valid bits: c < 32, or already appended
      syms = entry_symbol(long_code);
      meta = entry_meta(long_code);
      DF11_KEEP_BRANCH();
    }
    uint32_t k = (meta >> 8) & 0xffu;
    if (k > rem) {                      // the last lookup holds codes past the quota (k <= 4, so rem < 4)
      syms &= (1u << (8u * rem)) - 1u;
      k = rem;
    }
    LdsBytes word = stage + (~minus_pos & ~3u);            // (pos - 1) & ~3
    if (minus_pos & 3u) {               // a lookup that starts on a word boundary has nothing for the word before it
      or32_aligned(word, align_bytes(syms, 0u, minus_pos));
      DF11_KEEP_BRANCH();
    }
    or32_aligned(word + 4, align_bytes(0u, syms, minus_pos));
    minus_pos -= k;
    rem -= k;
    w <<= (meta & 63u);
    c += meta & 0xffu;
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

// ---- sub-blocks ------------------------------------------------------------------
// A sub-block is the 512 bytes of bitstream that one 64-lane wavefront decodes:
// 64 chunks, an eighth of a 4096-byte block.  The element index at which each
// sub-block's output starts is derived once per tensor (it depends only on the
// stream), which lets every wavefront work on its own, with no exchange between
// the wavefronts of a workgroup.
constexpr int kLanes = 64;
constexpr int kSubBytes = kLanes * kChunkBytes;          // 512
constexpr int kSubsPerBlock = kBlockBytes / kSubBytes;   // 8
constexpr int kMaxElemsPerSub = kSubBytes * 8;           // one-bit codes
constexpr int kGroup = 8;                                // elements per lane per write-out step

// Workspace derived once per tensor: header | decode tables | sub-block positions.
// A workspace is valid for the stream it was prepared from and for the library build
// that prepared it: the header records the layout's number and the stream's table count
// so that a dump of one can be told from another, but df11_decode does not read the
// header back (that would take a device read per call).
struct WorkspaceHeader {
  uint32_t magic;
  uint32_t n_blocks;
  uint32_t max_sub_elems;   // largest number of elements any sub-block produces
  uint32_t layout;          // kWorkspaceLayout of the build that wrote it
  uint32_t n_luts;          // rows of the stream's luts, the length row included
  uint32_t reserved[11];
};
constexpr uint32_t kWorkspaceLayout = 3;            // 3: fused 16-bit LUT rows follow the tables
constexpr uint32_t kWorkspaceMagic = 0x31314644u;   // "DF11"
constexpr int kWsTablesOffset = 64;
constexpr int kWsSubposOffset = kWsTablesOffset + kTablesBytes;
DF11_HD int64_t workspace_bytes(int64_t n_blocks) {
  return (kWsSubposOffset + 4 * (n_blocks * kSubsPerBlock + 1) + 15) & ~(int64_t)15;
}

// ---- search over the sub-block positions (row decode) -----------------------------
// Which sub-block holds output element `start`: the last entry of the ascending
// positions that is <= start.  The 64 lanes of a wavefront probe 64 evenly spaced
// entries of the remaining range at a time, so 2^24 entries take four dependent loads.
// The range [lo, hi) always holds the answer and its first entry is <= start (entry 0 of
// the positions is 0).
struct SubSearch {
  uint32_t lo, hi;
};
DF11_HD bool search_last_step(const SubSearch& r) { return r.hi - r.lo <= (uint32_t)kLanes; }
DF11_HD uint32_t search_stride(const SubSearch& r) {
  return search_last_step(r) ? 1u : (r.hi - r.lo + (uint32_t)kLanes - 1u) / (uint32_t)kLanes;
}
// Entry that `lane` probes, and whether it lies inside the range (a lane outside says no).
DF11_HD uint32_t search_probe(const SubSearch& r, uint32_t lane) { return r.lo + lane * search_stride(r); }
// `yes` lanes found their entry <= start: a run from lane 0, which is one of them (at
// least one is assumed, so that positions that do not ascend cannot lead anywhere odd).
// On the last step the answer is the range's `lo`.
DF11_HD SubSearch search_narrow(const SubSearch& r, uint32_t yes) {
  const uint32_t stride = search_stride(r);
  SubSearch n;
  n.lo = r.lo + ((yes ? yes : 1u) - 1u) * stride;
  n.hi = n.lo + stride < r.hi ? n.lo + stride : r.hi;
  return n;
}

// Where a sub-block lands.  The wavefront's staging area keeps the output's
// phase modulo 8 elements (staging index i holds output element a0 + i), so
// that 8-byte staging reads pair with 8-byte sign|mantissa loads and 16-byte
// BF16 stores.
struct SubPlan {
  int64_t a0;       // output index of staging index 0 (multiple of 8)
  uint32_t phase;   // staging index of the sub-block's first element, 0..7
  uint32_t n_out;   // elements produced (clamped to n_elements and to the staging capacity)
};

// Staging bytes one wavefront needs for sub-blocks of up to max_sub elements: the
// output phase (up to 7), the elements, and the 8 bytes that the word pair of a
// replayed lookup may cover past the last element; a multiple of 16.
constexpr int kStageSlack = 8;
DF11_HD int32_t stage_capacity(int32_t max_sub) {
  return ((max_sub + (kGroup - 1) + kStageSlack + 15) / 16) * 16;
}

DF11_HD SubPlan plan_sub(int64_t base, uint32_t total, int64_t n_elements, int32_t stage_cap) {
  SubPlan p;
  p.a0 = base & ~(int64_t)(kGroup - 1);
  p.phase = (uint32_t)(base - p.a0);
  int64_t end = base + (int64_t)total;
  if (end > n_elements) end = n_elements;
  int64_t n_out = end > base ? end - base : 0;
  const int64_t room = (int64_t)stage_cap - kStageSlack - (int64_t)p.phase;
  if (n_out > room) n_out = room;
  p.n_out = (uint32_t)n_out;
  return p;
}

// Staging bytes a sub-block may have touched, a multiple of 8: what has to be
// zero again before the next sub-block is replayed into the same area.
DF11_HD uint32_t stage_used(const SubPlan& p) {
  return (p.phase + p.n_out + (uint32_t)kStageSlack + 7u) & ~7u;
}

// How many of its `count` codes a thread with exclusive prefix `excl` decodes.
DF11_HD uint32_t thread_quota(uint32_t excl, uint32_t count, uint32_t n_out) {
  uint32_t my_end = excl + count;
  if (my_end > n_out) my_end = n_out;
  return my_end > excl ? my_end - excl : 0u;
}

// Four BF16 words from four exponent bytes E and four sign|mantissa bytes S:
// high bytes (S & 0x80) | (E >> 1), low bytes (E << 7) | (S & 0x7f), interleaved.
DF11_HD void merge4(uint32_t E, uint32_t S, uint32_t& out01, uint32_t& out23) {
  constexpr uint32_t kTop = 0x80808080u;   // bit 7 of every byte
  const uint32_t hi = (S & kTop) | ((E >> 1) & ~kTop);
  const uint32_t lo = ((E << 7) & kTop) | (S & ~kTop);
#if defined(__HIP_DEVICE_COMPILE__)
  out01 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);   // lo0 hi0 lo1 hi1
  out23 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);   // lo2 hi2 lo3 hi3
#else
  out01 = (lo & 0xffu) | ((hi & 0xffu) << 8) | ((lo & 0xff00u) << 8) | ((hi & 0xff00u) << 16);
  out23 = ((lo >> 16) & 0xffu) | ((hi >> 8) & 0xff00u) | ((lo >> 8) & 0xff0000u) | (hi & 0xff000000u);
#endif
}

// The write-out of a sub-block splits [phase, phase + n_out) into a head of
// fewer than 8 elements up to the first 8-aligned staging index, a body of
// whole 8-element groups, and a tail of fewer than 8 elements.
struct SubSpans {
  uint32_t head_begin, head_end;   // element-wise
  uint32_t body_begin, body_end;   // group indices (staging index / 8)
  uint32_t tail_begin, tail_end;   // element-wise
};

DF11_HD SubSpans spans_of(const SubPlan& p) {
  SubSpans s;
  const uint32_t first = p.phase, last = p.phase + p.n_out;
  s.head_begin = first;
  uint32_t up = (first + (uint32_t)kGroup - 1u) & ~(uint32_t)(kGroup - 1);
  s.head_end = up < last ? up : last;
  s.body_begin = s.head_end / (uint32_t)kGroup;       // only meaningful if a body exists
  s.body_end = last / (uint32_t)kGroup;
  if (s.body_end < s.body_begin) s.body_end = s.body_begin;
  const uint32_t body_last = s.body_end * (uint32_t)kGroup;
  s.tail_begin = body_last > s.head_end ? body_last : s.head_end;
  s.tail_end = last;
  return s;
}

// Eight BF16 words from 8 staging bytes `e` and 8 sign|mantissa bytes `m`.
DF11_HD U32x4 merge8(const U32x2& e, const U32x2& m) {
  U32x4 o;
  merge4(e.x, m.x, o.x, o.y);
  merge4(e.y, m.y, o.z, o.w);
  return o;
}

// Body group g: 8 staging bytes + 8 sign|mantissa bytes `m` -> 16 bytes of BF16.
DF11_HD void stream_group(uint32_t g, const SubPlan& p, ConstLdsBytes stage, const U32x2& m,
                          uint16_t* out) {
  const uint32_t s0 = g * (uint32_t)kGroup;
  store_as<U32x4>(out + p.a0 + s0, merge8(lds_load<U32x2>(stage + s0), m));
}

// One element of a head or tail (or of everything, for unaligned buffers).
DF11_HD void stream_element(uint32_t i, const SubPlan& p, ConstLdsBytes stage,
                            const uint8_t* sign_mantissa, uint16_t* out) {
  out[p.a0 + i] = merge(stage[i], sign_mantissa[p.a0 + i]);
}

}  // namespace df11
