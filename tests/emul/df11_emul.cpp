// Host emulation of the decode kernel's data flow, for bounds-checked testing
// without a GPU.  It calls the very functions the gfx950 kernel calls
// (dfloat11_amd/csrc/df11_core.h) in the same order -- table build, chunk
// fetch, count, exclusive prefix, staged emit, grouped stream-out -- one
// "thread" after another.  Every buffer is a heap copy of exactly the size the
// kernel is entitled to touch, so an AddressSanitizer build turns any
// out-of-range access in the shared logic into a test failure.
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../dfloat11_amd/csrc/df11_core.h"

using namespace df11;

namespace {
// Heap block of exactly n elements: malloc gives a 16-byte aligned start and,
// under AddressSanitizer, a red zone that begins right after the last byte.
template <class T>
struct Exact {
  T* p;
  explicit Exact(size_t n) : p(static_cast<T*>(malloc(n * sizeof(T) ? n * sizeof(T) : 1))) {}
  ~Exact() { free(p); }
  Exact(const Exact&) = delete;
};
}  // namespace

extern "C" int df11_emul_tables(const uint8_t* luts, int n_luts, uint8_t* tables) {
  const int n_rows = n_luts - 1 < kMaxDecodeRows ? n_luts - 1 : kMaxDecodeRows;
  std::vector<uint8_t> rows((size_t)(n_rows + 1) * 256);
  memcpy(rows.data(), luts, (size_t)n_rows * 256);
  memcpy(rows.data() + (size_t)n_rows * 256, luts + (size_t)(n_luts - 1) * 256, 256);
  Luts l{rows.data(), n_rows};
  for (uint32_t idx = 0; idx < (uint32_t)kTableEntries; ++idx) {
    uint32_t e[2];
    make_dec_entry(l, idx, e[0], e[1]);
    memcpy(tables + kDecOffset + 8 * idx, e, 8);
    tables[kCntTailOffset + idx] = make_cnt_tail_entry(l, idx);
  }
  for (uint32_t i = 0; i < (uint32_t)n_rows * 256u; ++i) {
    const uint16_t e = make_row_entry(l, i >> 8, i & 0xffu);
    memcpy(tables + kRowsOffset + 2 * i, &e, 2);
  }
  return 0;
}

// Host counterpart of df11_prepare: header, tables and the start index of every
// sub-block.  `ws` has workspace_bytes(n_blocks) bytes.  Returns the largest
// number of elements a sub-block produces.
extern "C" int df11_emul_prepare(const uint8_t* luts, const uint8_t* codes, const uint32_t* positions,
                                 const uint8_t* gaps, int n_luts, int64_t n_bytes, int64_t n_elements,
                                 uint8_t* ws) {
  const int64_t n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  const int n_rows = n_luts - 1 < kMaxDecodeRows ? n_luts - 1 : kMaxDecodeRows;
  memset(ws, 0, (size_t)workspace_bytes(n_blocks));
  df11_emul_tables(luts, n_luts, ws + kWsTablesOffset);
  // the passes read an exact-size copy of the part of the blob a decode loads
  Exact<uint8_t> blob((size_t)tables_bytes(n_rows));
  memcpy(blob.p, ws + kWsTablesOffset, (size_t)tables_bytes(n_rows));
  const Tables t{blob.p + kDecOffset, blob.p + kCntTailOffset};
  const Rows l{blob.p + kRowsOffset};
  std::vector<uint32_t> subpos((size_t)n_blocks * kSubsPerBlock + 1);
  uint32_t max_sub = 0;
  for (int64_t blk = 0; blk < n_blocks; ++blk) {
    int64_t start = positions[blk];
    for (int w = 0; w < kSubsPerBlock; ++w) {
      uint32_t total = 0;
      for (int lane = 0; lane < kLanes; ++lane) {
        const int64_t gid = (blk * kSubsPerBlock + w) * kLanes + lane;
        const Chunk c = fetch_chunk(codes, n_bytes, gid, false);
        total += count_chunk(t, l, c.hi, c.lo, c.next, gap_of(gaps, gid, n_blocks * kGapBytesPerBlock));
      }
      int64_t s0 = start < n_elements ? start : n_elements;
      int64_t e0 = start + total < n_elements ? start + total : n_elements;
      subpos[(size_t)(blk * kSubsPerBlock + w)] = (uint32_t)s0;
      if ((uint32_t)(e0 - s0) > max_sub) max_sub = (uint32_t)(e0 - s0);
      start += total;
    }
  }
  subpos[(size_t)n_blocks * kSubsPerBlock] = (uint32_t)n_elements;
  memcpy(ws + kWsSubposOffset, subpos.data(), subpos.size() * 4);
  WorkspaceHeader h{};
  h.magic = kWorkspaceMagic;
  h.n_blocks = (uint32_t)n_blocks;
  h.max_sub_elems = max_sub;
  h.layout = kWorkspaceLayout;
  h.n_luts = (uint32_t)n_luts;
  memcpy(ws, &h, sizeof h);
  return (int)max_sub;
}

// Same data arguments as df11_decode (include/df11.h), host pointers; `grid`
// plays gridDim.x (workgroups of eight wavefronts).  max_elems_per_sub <= 0
// selects the worst case, as in the library.
// The decode kernel's steps, for a whole stream (row_ids null: sub-blocks in the order
// the persistent grid takes them) or for the rows `row_ids` of the output matrix only
// (df11_decode_rows: `out` comes in holding what the caller's buffer held, and only the
// sub-blocks that overlap the rows are decoded into it).
template <int kMain>
static int emul_run(const uint8_t* luts, const uint8_t* codes, const uint8_t* sign_mantissa,
                    const uint32_t* positions, const uint8_t* gaps, uint16_t* out,
                    int n_luts, int64_t n_bytes, int64_t n_elements,
                    int max_elems_per_sub, int grid, int codes_misalign,
                    int out_misalign, int flags, const int64_t* row_ids, int64_t n_ids, int64_t row_elements) {
  if (max_elems_per_sub <= 0 || max_elems_per_sub > kMaxElemsPerSub) max_elems_per_sub = kMaxElemsPerSub;
  const int64_t n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  const int64_t n_subs = (n_bytes + kSubBytes - 1) / kSubBytes;
  const int stage_cap = stage_capacity(max_elems_per_sub);
  const int n_rows = n_luts - 1 < kMaxDecodeRows ? n_luts - 1 : kMaxDecodeRows;

  // exact-size copies of everything the kernel may read
  Exact<uint8_t> c_codes((size_t)n_bytes + codes_misalign);
  uint8_t* codes_p = c_codes.p + codes_misalign;
  memcpy(codes_p, codes, (size_t)n_bytes);
  Exact<uint8_t> c_sm((size_t)n_elements + out_misalign);
  uint8_t* sm_p = c_sm.p + out_misalign;
  memcpy(sm_p, sign_mantissa, (size_t)n_elements);
  Exact<uint32_t> c_pos((size_t)n_blocks);
  memcpy(c_pos.p, positions, (size_t)n_blocks * 4);
  Exact<uint8_t> c_gaps((size_t)n_blocks * kGapBytesPerBlock);
  memcpy(c_gaps.p, gaps, (size_t)n_blocks * kGapBytesPerBlock);
  Exact<uint16_t> c_out((size_t)n_elements + out_misalign);
  uint16_t* out_p = c_out.p + out_misalign;
  memset(c_out.p, 0xEE, ((size_t)n_elements + out_misalign) * 2);
  if (row_ids) memcpy(out_p, out, (size_t)n_elements * 2);
  Exact<uint8_t> ws((size_t)workspace_bytes(n_blocks));
  df11_emul_prepare(luts, codes_p, c_pos.p, c_gaps.p, n_luts, n_bytes, n_elements, ws.p);
  Exact<uint8_t> blob((size_t)tables_bytes(n_rows));   // what a workgroup copies into LDS
  memcpy(blob.p, ws.p + kWsTablesOffset, (size_t)tables_bytes(n_rows));
  // The staging area follows other data in the kernel's LDS (tables, other
  // wavefronts' areas): the replay may OR zero into the word before it.
  constexpr int kLeadIn = 16;
  Exact<uint8_t> stage_mem((size_t)kLeadIn + (size_t)stage_cap);
  memset(stage_mem.p, 0, (size_t)kLeadIn + (size_t)stage_cap);   // the kernel clears each wavefront's area once at start
  struct { uint8_t* p; } stage{stage_mem.p + kLeadIn};

  const Tables t{blob.p + kDecOffset, blob.p + kCntTailOffset};
  const Rows l{blob.p + kRowsOffset};
  const uint32_t* subpos = reinterpret_cast<const uint32_t*>(ws.p + kWsSubposOffset);
  const bool codes_aligned = (reinterpret_cast<uintptr_t>(codes_p) & 7) == 0;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(sm_p) & 7) == 0 &&
                      (reinterpret_cast<uintptr_t>(out_p) & 15) == 0;
  const int64_t n_gap_bytes = n_blocks * kGapBytesPerBlock;
  const int64_t stride = (int64_t)grid * kSubsPerBlock;

  std::vector<Chunk> chunk(kLanes);
  std::vector<uint32_t> gap(kLanes), count(kLanes), excl(kLanes);
  std::vector<ChunkSyms<kMain>> regs(kLanes);
  const bool force_two_pass = (flags & 1) != 0;   // exercise the fall-back route on any input
  auto do_sub = [&](int64_t sub) -> int {
    {
      // one decode per chunk into "registers"; a lane that ran out of slots counts the
      // rest of its chunk, and decodes that rest again once its offset is known
      for (int lane = 0; lane < kLanes; ++lane) {
        const int64_t gid = sub * kLanes + lane;
        chunk[lane] = fetch_chunk(codes_p, n_bytes, gid, codes_aligned);
        gap[lane] = gap_of(c_gaps.p, gid, n_gap_bytes);
        regs[lane] = decode_chunk_regs<kMain, true>(t, l, chunk[lane].hi, chunk[lane].lo, chunk[lane].next, gap[lane]);
      }
      uint32_t total = 0;
      for (int lane = 0; lane < kLanes; ++lane) {
        count[lane] = regs[lane].count;
        if (regs[lane].overflow)
          count[lane] += count_chunk(t, l, chunk[lane].hi, chunk[lane].lo, chunk[lane].next, regs[lane].resume);
        // the register route and the counting pass over the whole chunk must agree
        if (count[lane] != count_chunk(t, l, chunk[lane].hi, chunk[lane].lo, chunk[lane].next, gap[lane])) return 7;
        excl[lane] = total;
        total += count[lane];
      }
      const SubPlan p = plan_sub((int64_t)subpos[sub], total, n_elements, stage_cap);
      bool replay = !force_two_pass;
      for (int lane = 0; lane < kLanes; ++lane)
        replay = replay && thread_quota(excl[lane], count[lane], p.n_out) == count[lane];
      // Replay ORs into the staging area: it must be all zero here, which is the
      // previous sub-block's clear of stage_used() bytes and nothing else.
      for (int i = -kLeadIn; i < stage_cap; ++i)
        if (stage.p[i]) return 8;
      // Lanes run concurrently on the device, so no lane may rely on a later lane
      // repairing what it wrote.  Even sub-blocks write in ascending lane order,
      // odd ones in descending order: a store that strays into a neighbour's
      // bytes corrupts the result in one of the two.
      for (int k = 0; k < kLanes; ++k) {
        const int lane = (sub & 1) ? kLanes - 1 - k : k;
        const uint32_t quota = thread_quota(excl[lane], count[lane], p.n_out);
        const uint32_t at = (uint32_t)kLeadIn + p.phase + excl[lane];
        if (replay) {
          replay_chunk(regs[lane], stage_mem.p, at);
          if (regs[lane].overflow)
            emit_chunk(t, l, chunk[lane].hi, chunk[lane].lo, chunk[lane].next, regs[lane].resume,
                       count[lane] - regs[lane].count, stage_mem.p, at + regs[lane].count);
        } else {
          emit_chunk(t, l, chunk[lane].hi, chunk[lane].lo, chunk[lane].next, gap[lane], quota, stage_mem.p, at);
        }
      }
      const SubSpans sp = spans_of(p);
      if (vec_ok) {
        for (uint32_t i = sp.head_begin; i < sp.head_end; ++i) stream_element(i, p, stage.p, sm_p, out_p);
        for (uint32_t g = sp.body_begin; g < sp.body_end; ++g)
          stream_group(g, p, stage.p, load_as<U32x2>(sm_p + p.a0 + (int64_t)g * kGroup), out_p);
        for (uint32_t i = sp.tail_begin; i < sp.tail_end; ++i) stream_element(i, p, stage.p, sm_p, out_p);
      } else {
        for (uint32_t i = p.phase; i < p.phase + p.n_out; ++i) stream_element(i, p, stage.p, sm_p, out_p);
      }
      memset(stage.p, 0, stage_used(p));
    }
    return 0;
  };
  if (!row_ids) {
    for (int64_t wave_gid = 0; wave_gid < stride; ++wave_gid)
      for (int64_t sub = wave_gid; sub < n_subs; sub += stride)
        if (int rc = do_sub(sub)) return rc;
  } else {
    // as decode_kernel_rows: per id, the sub-block that holds the row's first element
    // (64 lanes probing the positions at a time), then sub-blocks until one starts past the row
    const uint32_t n_entries = (uint32_t)(n_blocks * kSubsPerBlock + 1);
    const int64_t n_rows_total = row_elements > 0 ? n_elements / row_elements : 0;
    Exact<uint32_t> pos_copy((size_t)n_entries);
    memcpy(pos_copy.p, subpos, (size_t)n_entries * 4);
    for (int64_t i = 0; i < n_ids; ++i) {
      const int64_t id = row_ids[i];
      if (id < 0 || id >= n_rows_total) continue;
      const int64_t first = id * row_elements, end = first + row_elements;
      SubSearch r{0u, n_entries};
      uint32_t s0;
      for (;;) {
        const bool last = search_last_step(r);
        uint32_t yes = 0;
        for (uint32_t lane = 0; lane < (uint32_t)kLanes; ++lane) {
          const uint32_t probe = search_probe(r, lane);
          if (probe < r.hi && pos_copy.p[probe] <= (uint32_t)first) ++yes;
        }
        r = search_narrow(r, yes);
        if (last) { s0 = r.lo; break; }
      }
      if (!(pos_copy.p[s0] <= (uint32_t)first && (s0 + 1 >= n_entries || pos_copy.p[s0 + 1] > (uint32_t)first)))
        return 9;   // the search must land on the sub-block that holds the element
      for (int64_t s = s0; s < n_subs; ++s) {
        if ((int64_t)pos_copy.p[s] >= end) break;
        if (int rc = do_sub(s)) return rc;
      }
    }
  }
  memcpy(out, out_p, (size_t)n_elements * 2);
  return 0;
}

// flags: bit 0 forces the two-pass route on every sub-block; bits 8-9 select the
// compilation by its register slots (0: the usual one, 1: the fewest, 2: short codes).
#define DF11_EMUL_DISPATCH(...)                                                   \
  switch ((flags >> 8) & 3) {                                                     \
    case 1: return emul_run<kMainSlotsFew>(__VA_ARGS__);                          \
    case 2: return emul_run<kMainSlotsShortCodes>(__VA_ARGS__);                   \
    default: return emul_run<kMainSlotsUsual>(__VA_ARGS__);                       \
  }

extern "C" int df11_emul_decode(const uint8_t* luts, const uint8_t* codes, const uint8_t* sign_mantissa,
                                const uint32_t* positions, const uint8_t* gaps, uint16_t* out,
                                int n_luts, int64_t n_bytes, int64_t n_elements,
                                int max_elems_per_sub, int grid, int codes_misalign,
                                int out_misalign, int flags) {
  DF11_EMUL_DISPATCH(luts, codes, sign_mantissa, positions, gaps, out, n_luts, n_bytes, n_elements, max_elems_per_sub,
                     grid, codes_misalign, out_misalign, flags, nullptr, 0, 0)
}

// Host counterpart of df11_decode_rows; `out` holds the caller's buffer on entry.
extern "C" int df11_emul_decode_rows(const uint8_t* luts, const uint8_t* codes, const uint8_t* sign_mantissa,
                                     const uint32_t* positions, const uint8_t* gaps, uint16_t* out,
                                     int n_luts, int64_t n_bytes, int64_t n_elements, int max_elems_per_sub,
                                     const int64_t* row_ids, int64_t n_ids, int64_t row_elements) {
  if (!row_ids || row_elements <= 0) return 1;
  const int flags = 0;
  DF11_EMUL_DISPATCH(luts, codes, sign_mantissa, positions, gaps, out, n_luts, n_bytes, n_elements, max_elems_per_sub,
                     1, 0, 0, flags, row_ids, n_ids, row_elements)
}

#ifdef DF11_EMUL_MAIN
// Stand-alone driver (built with AddressSanitizer): reads one case from a file
//   i64 n_luts, n_bytes, n_elements, n_blocks, max_elems, grid, codes_misalign, out_misalign, flags
//   (flags bit 2: df11_decode_rows for a fixed choice of rows instead of the whole stream)
//   luts | codes | sign_mantissa | positions (n_blocks u32) | gaps
// and writes the decoded u16 words to the output file.
#include <cstdio>
int main(int argc, char** argv) {
  if (argc != 3) return 2;
  FILE* f = fopen(argv[1], "rb");
  if (!f) return 2;
  int64_t h[9];
  if (fread(h, 8, 9, f) != 9) return 2;
  const int64_t n_luts = h[0], n_bytes = h[1], n_elements = h[2], n_blocks = h[3];
  Exact<uint8_t> luts((size_t)n_luts * 256), codes((size_t)n_bytes), sm((size_t)n_elements);
  Exact<uint32_t> pos((size_t)n_blocks);
  Exact<uint8_t> gaps((size_t)n_blocks * kGapBytesPerBlock);
  Exact<uint16_t> out((size_t)n_elements);
  bool ok = fread(luts.p, 1, (size_t)n_luts * 256, f) == (size_t)n_luts * 256 &&
            fread(codes.p, 1, (size_t)n_bytes, f) == (size_t)n_bytes &&
            fread(sm.p, 1, (size_t)n_elements, f) == (size_t)n_elements &&
            fread(pos.p, 4, (size_t)n_blocks, f) == (size_t)n_blocks &&
            fread(gaps.p, 1, (size_t)n_blocks * kGapBytesPerBlock, f) == (size_t)n_blocks * kGapBytesPerBlock;
  fclose(f);
  if (!ok) return 2;
  int rc;
  if (h[8] & 4) {
    // rows mode: the output as a matrix of seven rows (the rest of the elements belong to
    // no row), rows 6, 0, 3 and 3 again and three numbers outside it, into a buffer of 0xEEEE
    const int64_t row_elements = n_elements / 7 > 0 ? n_elements / 7 : 1;
    Exact<int64_t> ids(7);
    const int64_t want[7] = {6, 0, 3, 3, -1, 7 + n_elements, 99};
    memcpy(ids.p, want, sizeof want);
    memset(out.p, 0xEE, (size_t)n_elements * 2);
    rc = df11_emul_decode_rows(luts.p, codes.p, sm.p, pos.p, gaps.p, out.p, (int)n_luts, n_bytes, n_elements,
                               (int)h[4], ids.p, 7, row_elements);
  } else {
    rc = df11_emul_decode(luts.p, codes.p, sm.p, pos.p, gaps.p, out.p, (int)n_luts, n_bytes,
                          n_elements, (int)h[4], (int)h[5], (int)h[6], (int)h[7], (int)h[8]);
  }
  if (rc) return 3;
  FILE* g = fopen(argv[2], "wb");
  if (!g) return 2;
  fwrite(out.p, 2, (size_t)n_elements, g);
  fclose(g);
  return 0;
}
#endif
