// gfx950 kernels and C-ABI for DF11 stream decode.
//
// Unit of work: a sub-block, the 512 bytes of bitstream (64 chunks of 8 bytes)
// that one 64-lane wavefront decodes.  The output index at which each sub-block
// starts is derived once per tensor by df11_prepare (it depends only on the
// compressed stream), so at decode time every wavefront is independent: no
// workgroup barrier and no exchange between wavefronts, only the decode tables
// in LDS are shared.  Workgroups of 512 threads walk the sub-blocks persistently
// (tables are copied into LDS once per workgroup).  Per sub-block a wavefront
//   1. takes its chunk (+4 bytes of look-ahead), gap and start index, all fetched
//      one sub-block ahead, and requests the sign|mantissa bytes it will need;
//   2. decodes each lane's chunk once (four-symbol table in LDS); the handful of
//      lookups a chunk needs stay in registers, and their count is the lane's
//      number of codes;
//   3. turns the 64 counts into exclusive offsets with a DPP scan;
//   4. replays the lookups from registers into its private, zeroed LDS staging
//      area, in output order, as aligned OR operations (chunks with too many
//      lookups for the registers fall back to counting first and decoding a
//      second time);
//   5. streams the staging area out: 8 exponent bytes (LDS) + 8 sign|mantissa
//      bytes -> one 16-byte BF16 store per lane, contiguous across the wavefront,
//      in batches of 64 lanes that start on 256-byte lines of the output.
// The kernel is bound by HBM; the decode (vector instructions for a little over
// half of the memory time on weight-like streams) is hidden under it with two to
// four workgroups per CU (the launch plans further down).  df11_decode_rows runs
// the same steps on the sub-blocks that hold given rows of the output only.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../include/df11.h"
#include "df11_core.h"

namespace {

using namespace df11;

thread_local hipError_t g_last_hip = hipSuccess;

inline int hip_fail(hipError_t e) {
  g_last_hip = e;
  return DF11_ERR_HIP;
}

constexpr int kWavesPerGroup = kThreads / kLanes;   // 8
constexpr int kLdsSkip = 16;   // decode_kernel's LDS layout starts at this address of the workgroup's allocation

// ---------------------------------------------------------------------------
// Wavefront inclusive scan with DPP (row shifts inside rows of 16 lanes, then
// row broadcasts across the four rows of the 64-lane wavefront).
// ---------------------------------------------------------------------------
template <int kCtrl, int kRowMask, int kBankMask, bool kBoundCtrl>
__device__ __forceinline__ uint32_t dpp_add(uint32_t v) {
  return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, kRowMask, kBankMask, kBoundCtrl);
}

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  v = dpp_add<0x111, 0xf, 0xf, true>(v);    // row_shr:1
  v = dpp_add<0x112, 0xf, 0xf, true>(v);    // row_shr:2
  v = dpp_add<0x114, 0xf, 0xf, true>(v);    // row_shr:4
  v = dpp_add<0x118, 0xf, 0xf, true>(v);    // row_shr:8
  v = dpp_add<0x142, 0xa, 0xf, false>(v);   // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xc, 0xf, false>(v);   // row_bcast:31 into rows 2 and 3
  return v;
}

__device__ __forceinline__ bool wave_all(bool pred) {
  return __builtin_amdgcn_ballot_w64(pred) == __builtin_amdgcn_ballot_w64(true);
}

__device__ __forceinline__ uint32_t wave_total(uint32_t inclusive) {
  return (uint32_t)__builtin_amdgcn_readlane((int)inclusive, 63);
}

// Copies the byte LUT rows a pointer can reach, then the length row, into LDS
// (table construction reads them; the decode reads the fused rows it writes).
__device__ __forceinline__ void stage_rows(const uint8_t* __restrict__ luts, int n_luts, int n_rows,
                                           uint8_t* rows, int tid, int n_threads) {
  for (int i = tid; i < n_rows * 256; i += n_threads) rows[i] = luts[i];
  for (int i = tid; i < 256; i += n_threads) rows[n_rows * 256 + i] = luts[(int64_t)(n_luts - 1) * 256 + i];
}

// ---------------------------------------------------------------------------
// Prepare, step 1: decode tables + header.  One thread per table index.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void build_tables_kernel(const uint8_t* __restrict__ luts, int n_luts,
                                                           uint8_t* __restrict__ ws, uint32_t n_blocks) {
  __shared__ uint8_t rows[(kMaxDecodeRows + 1) * 256];
  const int n_rows = min(n_luts - 1, kMaxDecodeRows);
  stage_rows(luts, n_luts, n_rows, rows, threadIdx.x, blockDim.x);
  __syncthreads();
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (uint32_t)kTableEntries) return;
  const Luts l{rows, n_rows};
  uint32_t syms, meta;
  make_dec_entry(l, idx, syms, meta);
  uint8_t* tables = ws + kWsTablesOffset;
  reinterpret_cast<uint2*>(tables + kDecOffset)[idx] = make_uint2(syms, meta);
  tables[kCntTailOffset + idx] = make_cnt_tail_entry(l, idx);
  uint16_t* fused = reinterpret_cast<uint16_t*>(tables + kRowsOffset);
  for (uint32_t i = idx; i < (uint32_t)n_rows * 256u; i += (uint32_t)kTableEntries)
    fused[i] = make_row_entry(l, i >> 8, i & 0xffu);
  if (idx < sizeof(WorkspaceHeader) / 4) {
    uint32_t v = 0;
    if (idx == 0) v = kWorkspaceMagic;
    if (idx == 1) v = n_blocks;
    if (idx == 3) v = kWorkspaceLayout;
    if (idx == 4) v = (uint32_t)n_luts;
    reinterpret_cast<uint32_t*>(ws)[idx] = v;   // max_sub_elems starts at 0
  }
}

// ---------------------------------------------------------------------------
// Prepare, step 2: where each sub-block's output starts.  One workgroup per
// 4096-byte block at a time: count per lane, totals per wavefront, offsets from
// the block's own output position.
// ---------------------------------------------------------------------------
struct IndexArgs {
  const uint8_t* codes;
  const uint32_t* positions;
  const uint8_t* gaps;
  uint8_t* ws;
  int64_t n_bytes;
  int64_t n_elements;
  int64_t n_blocks;
  int32_t n_luts;
  int32_t codes_aligned;
};

__global__ __launch_bounds__(kThreads) void index_kernel(const IndexArgs a) {
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_rows = min(a.n_luts - 1, kMaxDecodeRows);
  const LdsBytes lds_tables = (LdsBytes)lds;
  uint32_t* wave_sums = reinterpret_cast<uint32_t*>(lds + kTablesBytes);
  {
    const uint4* src = reinterpret_cast<const uint4*>(a.ws + kWsTablesOffset);
    uint4* dst = reinterpret_cast<uint4*>(lds);
    for (int i = tid; i < tables_bytes(n_rows) / 16; i += kThreads) dst[i] = src[i];
  }
  __syncthreads();
  const Tables t{lds_tables + kDecOffset, lds_tables + kCntTailOffset};
  const Rows l{lds_tables + kRowsOffset};
  const int64_t n_gap_bytes = a.n_blocks * kGapBytesPerBlock;
  uint32_t* subpos = reinterpret_cast<uint32_t*>(a.ws + kWsSubposOffset);
  uint32_t my_max = 0;
  for (int64_t blk = blockIdx.x; blk < a.n_blocks; blk += gridDim.x) {
    const int64_t gid = blk * kThreads + tid;
    const Chunk c = fetch_chunk(a.codes, a.n_bytes, gid, a.codes_aligned != 0);
    const uint32_t gap = gap_of(a.gaps, gid, n_gap_bytes);
    const uint32_t count = count_chunk(t, l, c.hi, c.lo, c.next, gap);
    const uint32_t incl = wave_inclusive_scan(count);
    if (lane == 63) wave_sums[wave] = incl;
    __syncthreads();
    if (tid < kWavesPerGroup) {
      int64_t start = (int64_t)a.positions[blk];
      for (int wv = 0; wv < tid; ++wv) start += wave_sums[wv];
      int64_t end = start + wave_sums[tid];
      if (start > a.n_elements) start = a.n_elements;
      if (end > a.n_elements) end = a.n_elements;
      subpos[blk * kSubsPerBlock + tid] = (uint32_t)start;
      my_max = max(my_max, (uint32_t)(end - start));
    }
    __syncthreads();   // wave_sums is rewritten by the next block
  }
  if (blockIdx.x == 0 && tid == 0) subpos[a.n_blocks * kSubsPerBlock] = (uint32_t)a.n_elements;
  if (tid < kWavesPerGroup && my_max)
    atomicMax(&reinterpret_cast<WorkspaceHeader*>(a.ws)->max_sub_elems, my_max);
}

// ---------------------------------------------------------------------------
// Decode kernel.
// LDS layout (dynamic): tables | the fused LUT rows that exist | 8 staging areas
//
// Everything that is the same for the 64 lanes of a wavefront (sub-block index,
// output position, plan of the write-out) is kept wavefront-uniform on purpose,
// so that it lives in scalar registers and costs no vector instructions; global
// addresses are a uniform 64-bit base plus a 32-bit lane offset.
// ---------------------------------------------------------------------------
// A zero the compiler cannot see through, held in a vector register: adding it to
// a uniform index keeps the access a vector load.
__device__ __forceinline__ uint32_t opaque_vector_zero() {
  uint32_t z;
  asm volatile("v_mov_b32 %0, 0" : "=v"(z));
  return z;
}

// Two consecutive 32-bit words at a 4-byte aligned address.
__device__ __forceinline__ U32x2 load_as_unaligned_pair(const uint32_t* p) {
  U32x2 v;
  v.x = p[0];
  v.y = p[1];
  return v;
}

// Marks loaded values as used at this point of the program, so that the wait for
// their arrival is placed here and not at their first real use.
__device__ __forceinline__ void claim(uint32_t& v) { asm volatile("" : "+v"(v)); }
template <class... T>
__device__ __forceinline__ void claim(uint32_t& v, T&... rest) {
  claim(v);
  claim(rest...);
}

// Streaming access: the output is written once and, within one decode, the
// bitstream and the sign|mantissa bytes are read once, so they bypass cache
// retention (nontemporal): worth 5-8 % on a large stream (plain stores: 145 vs
// 133 us on the 218 M-element block; plain loads: 387 vs 368 us on 622 M
// elements).  kStreaming = false reads with plain loads instead, for the small
// streams of the `wide` plan: what a small stream's module reads may still sit in
// the 256 MB memory-side cache from the previous forward pass (a 17 M-element
// weight decodes in 13.1-13.8 us instead of 14.8-15.4 us then), and when it does
// not the plain loads cost 1.5 % (16.3 vs 16.1 us with 24 copies decoded in turn).
typedef uint32_t V4u __attribute__((ext_vector_type(4)));
typedef uint32_t V2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_stream(uint16_t* p, const U32x4& v) {
  const V4u x = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(x, reinterpret_cast<V4u*>(p));
}
template <bool kStreaming>
__device__ __forceinline__ U32x2 load_stream(const uint8_t* p) {   // p 8-byte aligned
  const V2u v = kStreaming ? __builtin_nontemporal_load(reinterpret_cast<const V2u*>(p))
                           : *reinterpret_cast<const V2u*>(p);
  return U32x2{v.x, v.y};
}

struct DecodeSizes {
  int64_t n_bytes;
  int64_t n_elements;
  int64_t n_blocks;
  int64_t n_subs;         // sub-blocks that hold stream bytes: ceil(n_bytes / 512)
  int32_t n_luts;
  int32_t stage_cap;      // bytes of staging per wavefront, multiple of 16
  int32_t codes_aligned;  // codes pointer is 8-byte aligned
  int32_t vec_ok;         // sign_mantissa 8-byte aligned and out 16-byte aligned
};

// kPrefetch (template parameter of the decode body): body groups per lane whose
// sign|mantissa bytes are requested a whole decode early; the remaining groups of
// a sub-block load theirs between the stores.  How many to request early and how
// many wavefronts to keep resident go together and depend on the stream (see the
// launch plans next to the kernels).
constexpr int kBatchAlignGroups = 16;   // batches of 64 groups start on multiples of 16 groups (256 B of output)

__device__ __forceinline__ uint32_t uniform(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
}

// Inputs of one sub-block exactly as loaded: nothing here is computed on, so
// requesting them one sub-block ahead never waits for them.
struct SubInputs {
  uint32_t d0, d1, d2;   // bytes [0,4), [4,8), [8,12) of the lane's chunk, little-endian words
  uint32_t gap_raw;      // two bytes of the packed gaps, little-endian
  uint32_t base;         // first output element (same in every lane)
  uint32_t end_hint;     // first output element of the next sub-block (same in every lane)
};

// Bytes [8*lane, 8*lane + 12) of sub-block `sub` (uniform), its two gap bytes and
// its output position.  gap_byte: lane's byte offset inside the sub-block's 40
// bytes of gaps, chosen so that byte + 1 stays inside them.
template <bool kStreaming>
__device__ __forceinline__ SubInputs fetch_sub(const uint8_t* __restrict__ codes,
                                               const uint8_t* __restrict__ gaps,
                                               const uint32_t* __restrict__ subpos,
                                               const DecodeSizes& z, int64_t sub, uint32_t lane,
                                               uint32_t gap_byte, uint32_t vector_zero) {
  SubInputs in;
  const int64_t sub_off = sub * kSubBytes;                       // uniform
  if (z.codes_aligned && sub_off + kSubBytes + 4 <= z.n_bytes) {   // uniform: whole sub-block + look-ahead in range
    const uint8_t* p = codes + sub_off + lane * (uint32_t)kChunkBytes;
    const U32x2 v = load_stream<kStreaming>(p);
    in.d0 = v.x;
    in.d1 = v.y;
    in.d2 = load_as<uint32_t>(p + 8);
  } else {
    const Chunk c = fetch_chunk(codes, z.n_bytes, sub * kLanes + lane, false);
    in.d0 = __builtin_bswap32(c.hi);
    in.d1 = __builtin_bswap32(c.lo);
    in.d2 = __builtin_bswap32(c.next);
  }
  uint16_t g16;
  __builtin_memcpy(&g16, gaps + sub * (kLanes * 5 / 8) + gap_byte, 2);   // unaligned 2-byte load
  in.gap_raw = g16;
  // Loaded per lane although the index is uniform: a scalar load would share its
  // wait counter with the LDS lookups and stall the first of them.  The value is
  // made uniform where it is consumed, not here: that would wait for the load one
  // sub-block too early.
  const U32x2 pos = load_as_unaligned_pair(subpos + sub + vector_zero);
  in.base = pos.x;
  in.end_hint = pos.y;
  return in;
}

// Rows of a matrix to decode (decode_kernel_rows): the elements
// [id * row_elements, (id + 1) * row_elements) of the stream's output for each id.
struct RowsArgs {
  const int64_t* ids;
  int64_t n_ids;
  int64_t row_elements;
};

// Index of the sub-block that holds output element `start` (< n_elements): the last
// entry of the ascending `subpos` (n_entries of them, the first is 0) that is <= start
// (SubSearch in df11_core.h).  The result is wavefront-uniform.
__device__ __forceinline__ uint32_t find_sub(const uint32_t* __restrict__ subpos, uint32_t n_entries,
                                             uint32_t start, uint32_t lane) {
  SubSearch r{0u, n_entries};
  for (;;) {
    const bool last = search_last_step(r);
    const uint32_t probe = search_probe(r, lane);
    const bool le = probe < r.hi && subpos[probe] <= start;
    r = search_narrow(r, (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(le)));
    if (last) return r.lo;
  }
}

template <int kPrefetchGroups, bool kStreaming, bool kPhasePriority, bool kConstantLdsBase, int kMain, bool kResume,
          bool kRows = false>
__device__ __forceinline__ void decode_body(
    const uint8_t* __restrict__ codes,
    const uint8_t* __restrict__ sign_mantissa, const uint8_t* __restrict__ gaps,
    uint16_t* __restrict__ out, const uint8_t* __restrict__ ws, const DecodeSizes z,
    const RowsArgs rows = RowsArgs{}) {
  // The decode kernels have no static LDS, so their dynamic LDS starts at address 0 of the
  // workgroup's allocation (the host checks the kernels' static size before the
  // first launch).  Spelling the base as a constant instead of the symbol of an
  // extern array lets the compiler fold it into the offset field of every LDS
  // instruction: the symbol costs one vector add per table lookup and staging
  // access.  The first kLdsSkip bytes stay unused (address 0 would read as null).
  // One compilation (`portable`) takes the base from the symbol all the same: it is
  // what runs if a toolchain ever gives the other kernels LDS of its own.
  extern __shared__ __align__(16) uint8_t dynamic_lds[];
  const LdsBytes lds = kConstantLdsBase ? reinterpret_cast<LdsBytes>((uintptr_t)kLdsSkip)
                                        : (LdsBytes)dynamic_lds + kLdsSkip;
  const int tid = threadIdx.x;
  const uint32_t lane = tid & 63;
  const uint32_t wave = uniform(tid >> 6);
  const int n_rows = min(z.n_luts - 1, kMaxDecodeRows);
  const LdsBytes lds_tables = lds;
  const uint32_t stage_offset = (uint32_t)tables_bytes(n_rows) + wave * (uint32_t)z.stage_cap;   // multiple of 16
  const LdsBytes stage = lds + stage_offset;
  const uint32_t* __restrict__ subpos = reinterpret_cast<const uint32_t*>(ws + kWsSubposOffset);
  // Lane constants of the 5-bit gap: two bytes starting at gap_byte hold it,
  // gap_shift positions it.  Lane 63's field ends its sub-block's gap bytes, so
  // its window starts one byte early and never reaches past them.
  const uint32_t gap_bit = lane * 5u;
  const uint32_t gap_byte = min(gap_bit >> 3, (uint32_t)(kLanes * 5 / 8 - 2));
  const uint32_t gap_shift = 11u - (gap_bit - 8u * gap_byte);
  int64_t sub = (int64_t)blockIdx.x * kWavesPerGroup + wave;   // uniform
  const uint32_t vzero = opaque_vector_zero();
  // The first sub-block's inputs are requested before the tables are copied, so
  // that their latency overlaps with that of the copy.
  SubInputs held{};
  if (!kRows && sub < z.n_subs) held = fetch_sub<kStreaming>(codes, gaps, subpos, z, sub, lane, gap_byte, vzero);
  {
    const uint4* src = reinterpret_cast<const uint4*>(ws + kWsTablesOffset);
    for (int i = tid; i < tables_bytes(n_rows) / 16; i += kThreads) lds_store<uint4>(lds_tables + 16 * i, src[i]);
  }
  // Replayed symbols are ORed into the staging area, which therefore starts out
  // zero and is cleared again after every sub-block.
  for (uint32_t i = lane * 8u; i < (uint32_t)z.stage_cap; i += kLanes * 8u) lds_store<U32x2>(stage + i, U32x2{0, 0});
  __syncthreads();   // the only workgroup barrier: tables are read-only from here on

  const Tables t{lds_tables + kDecOffset, lds_tables + kCntTailOffset};
  const Rows l{lds_tables + kRowsOffset};
  const bool vec_ok = z.vec_ok != 0;
  const int64_t stride = (int64_t)gridDim.x * kWavesPerGroup;
  if (!kRows && sub >= z.n_subs) return;
  claim(held.d0, held.d1, held.d2, held.gap_raw, held.base, held.end_hint);   // see the claim inside the step

  // The instruction arbiter prefers the oldest wavefront of a SIMD, so with equal
  // shares of work the wavefronts launched first would finish well before the
  // others and leave the CU half empty towards the end.  Each wavefront therefore
  // walks through the four priority levels, one step per sub-block, from a
  // starting point given by its slot on the SIMD: over time every wavefront gets
  // the same share and all of them finish together.
  // A stream of few sub-blocks per wavefront has no long run to even out; there
  // (kPhasePriority) the priority follows the phase instead: lowest while a
  // wavefront decodes, highest while it writes out and requests the next
  // sub-block's inputs, so that stores and loads are issued as soon as they can be
  // and the decodes of the other wavefronts fill the gaps.
  uint32_t turn = __builtin_amdgcn_s_getreg((3 << 11) | 4);   // HW_ID.WAVE_ID, the slot on the SIMD
  // One sub-block, whose inputs `cur` holds; returns the inputs of sub-block `next_sub`,
  // requested on the way if `fetch_next` says that it exists.
  auto step = [&](const SubInputs& cur, bool fetch_next, int64_t next_sub) __attribute__((always_inline)) -> SubInputs {
    if (!kPhasePriority) {
      switch (turn++ & 3u) {   // s_setprio takes an immediate
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
      }
    }
    // ---- requests whose latency the two decode passes hide: the next
    // sub-block's inputs and this one's sign|mantissa bytes
    SubInputs nxt = cur;
    if (fetch_next) nxt = fetch_sub<kStreaming>(codes, gaps, subpos, z, next_sub, lane, gap_byte, vzero);

    const uint32_t base = uniform(cur.base);
    const uint32_t a0 = base & ~(uint32_t)(kGroup - 1);
    const uint32_t n_total = (uint32_t)z.n_elements;          // < 2^32, checked by the host
    const uint32_t end_hint = min(uniform(cur.end_hint), n_total);
    const uint32_t hint_len = end_hint > a0 ? end_hint - a0 : 0u;   // staging index one past the hinted end
    const uint32_t first_body = (base != a0) ? 1u : 0u;       // group 0 is a partial head unless aligned
    const uint8_t* sm0 = sign_mantissa + a0;                  // uniform bases
    uint16_t* out0 = out + a0;
    // Lanes are assigned to groups so that every 64-lane batch starts on a 256-byte
    // boundary of the output (128 bytes of sign|mantissa): the first `skew` lanes of
    // the first batch stay idle.  A sub-block starts at an arbitrary element, and
    // 1 KB stores that straddle lines cost 9 % of the kernel's time on fresh data.
    const uint32_t skew = ((a0 >> 3) + first_body) & (uint32_t)(kBatchAlignGroups - 1);
    U32x2 m[kPrefetchGroups];
#pragma unroll
    for (int k = 0; k < kPrefetchGroups; ++k) {
      m[k] = U32x2{0, 0};
      const uint32_t s0 = (first_body + lane + (uint32_t)(kLanes * k) - skew) * (uint32_t)kGroup;
      if (vec_ok && (k > 0 || lane >= skew) && s0 + (uint32_t)kGroup <= hint_len) m[k] = load_stream<kStreaming>(sm0 + s0);
    }
    // The ragged ends, fewer than 8 elements each: lanes 0..7 take the head, lanes
    // 8..15 the tail, one element per lane, its sign|mantissa byte requested now.
    const uint32_t phase0 = base - a0;
    const uint32_t head_end_hint = phase0 ? min((uint32_t)kGroup, hint_len) : 0u;
    const uint32_t tail_begin_hint = max(hint_len & ~(uint32_t)(kGroup - 1), head_end_hint);
    const uint32_t edge_hint = lane < (uint32_t)kGroup ? phase0 + lane : tail_begin_hint + lane - (uint32_t)kGroup;
    const bool edge_hint_ok = vec_ok && lane < 2u * kGroup &&
                              (lane < (uint32_t)kGroup ? edge_hint < head_end_hint : edge_hint < hint_len);
    uint32_t edge_byte = 0;
    if (edge_hint_ok) edge_byte = sm0[edge_hint];

    // ---- decode, and the exclusive offsets inside the wavefront
    if (kPhasePriority) __builtin_amdgcn_s_setprio(0);
    const Chunk c{__builtin_bswap32(cur.d0), __builtin_bswap32(cur.d1), __builtin_bswap32(cur.d2)};
    const uint32_t gap_word = __builtin_bswap32(cur.gap_raw) >> 16;   // the two bytes, big-endian
    const uint32_t gap = (gap_word >> gap_shift) & 31u;
    // One decode per chunk, results held in registers.  A lane that ran out of
    // register slots counts the rest of its chunk now and decodes that rest a second
    // time once its offset is known.  If some lane may not write all its symbols (end
    // of the tensor, staging smaller than the sub-block), the wavefront decodes
    // everything a second time instead, up to each lane's quota.
    const ChunkSyms<kMain> cs = decode_chunk_regs<kMain, kResume>(t, l, c.hi, c.lo, c.next, gap);
    // (The compilations for eight wavefronts per SIMD have no register left for the place
    // where a lane's rest starts: there a wavefront with such a lane counts and decodes
    // whole chunks again.)
    const bool redo_all = !kResume && !wave_all(!cs.overflow);
    uint32_t count = cs.count;
    if (redo_all) {
      count = count_chunk(t, l, c.hi, c.lo, c.next, gap);
    } else if (kResume && cs.overflow) {
      count += count_chunk(t, l, c.hi, c.lo, c.next, cs.resume);
      DF11_KEEP_BRANCH();
    }
    const uint32_t incl = wave_inclusive_scan(count);
    const uint32_t total = wave_total(incl);                  // uniform
    const uint32_t excl = incl - count;

    // ---- symbols to their place in the staging area, in output order
    const SubPlan p = plan_sub((int64_t)base, total, z.n_elements, z.stage_cap);   // uniform
    const uint32_t quota = thread_quota(excl, count, p.n_out);
    if (!redo_all && wave_all(quota == count)) {
      replay_chunk(cs, lds, stage_offset + p.phase + excl);   // one base for all: the wavefront's offset rides in the index
      if (kResume && cs.overflow) {
        emit_chunk(t, l, c.hi, c.lo, c.next, cs.resume, count - cs.count, lds, stage_offset + p.phase + excl + cs.count);
        DF11_KEEP_BRANCH();
      }
    } else {
      emit_chunk(t, l, c.hi, c.lo, c.next, gap, quota, lds, stage_offset + p.phase + excl);
    }
    // Staging is exchanged between the lanes of one wavefront only; its LDS
    // operations execute in order, the fence keeps the compiler from reordering.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- stream out
    if (kPhasePriority) __builtin_amdgcn_s_setprio(3);
    // Vector loads and stores share one in-order completion counter on this
    // hardware, so the first use of a loaded value after a store waits for that
    // store to reach memory.  Every value requested above is therefore claimed
    // here, before the first store of this sub-block is issued; by now those
    // loads are a whole decode old and the wait costs nothing.
    claim(nxt.d0, nxt.d1, nxt.d2, nxt.gap_raw, nxt.base, nxt.end_hint);
#pragma unroll
    for (int k = 0; k < kPrefetchGroups; ++k) claim(m[k].x, m[k].y);
    claim(edge_byte);

    const SubSpans sp = spans_of(p);                          // uniform
    if (vec_ok && p.phase + p.n_out == hint_len) {
      // The hint was exact (it always is for a well-formed workspace): every
      // sign|mantissa byte of the first kPrefetchGroups x 64 groups and of the ragged
      // ends is in registers.
      U32x4 o[kPrefetchGroups];
      uint32_t g = sp.body_begin + lane - skew;   // below body_begin (or wrapped) for the idle lanes of batch 0
#pragma unroll
      for (int k = 0; k < kPrefetchGroups; ++k) {
        const uint32_t gk = g + (uint32_t)(kLanes * k);
        const bool on = (k > 0 || lane >= skew) && gk < sp.body_end;
        const uint32_t s0 = (on ? gk : 0u) * (uint32_t)kGroup;   // in range for idle lanes too
        o[k] = merge8(lds_load<U32x2>(stage + s0), m[k]);
      }
      const bool is_head = lane < (uint32_t)kGroup;
      const uint32_t edge = is_head ? sp.head_begin + lane : sp.tail_begin + lane - (uint32_t)kGroup;
      const bool edge_on = lane < 2u * kGroup && edge < (is_head ? sp.head_end : sp.tail_end);
      const uint16_t edge_word = merge(stage[edge_on ? edge : 0u], edge_byte);
#pragma unroll
      for (int k = 0; k < kPrefetchGroups; ++k) {
        const uint32_t gk = g + (uint32_t)(kLanes * k);
        if ((k > 0 || lane >= skew) && gk < sp.body_end) store_stream(out0 + gk * (uint32_t)kGroup, o[k]);
      }
      if (edge_on) out0[edge] = edge_word;
      // the groups past the prefetched ones
      for (g += (uint32_t)(kLanes * kPrefetchGroups); g < sp.body_end; g += kLanes) {
        const uint32_t s0 = g * (uint32_t)kGroup;
        store_stream(out0 + s0, merge8(lds_load<U32x2>(stage + s0), load_as<U32x2>(sm0 + s0)));
      }
    } else if (vec_ok) {
      for (uint32_t i = sp.head_begin + lane; i < sp.head_end; i += kLanes) out0[i] = merge(stage[i], sm0[i]);
      for (uint32_t g = sp.body_begin + lane; g < sp.body_end; g += kLanes) {
        const uint32_t s0 = g * (uint32_t)kGroup;
        store_stream(out0 + s0, merge8(lds_load<U32x2>(stage + s0), load_as<U32x2>(sm0 + s0)));
      }
      for (uint32_t i = sp.tail_begin + lane; i < sp.tail_end; i += kLanes) out0[i] = merge(stage[i], sm0[i]);
    } else {
      for (uint32_t i = p.phase + lane; i < p.phase + p.n_out; i += kLanes)
        out0[i] = merge(stage[i], sm0[i]);
    }
    // Clear what this sub-block may have touched.  LDS operations of a wavefront
    // execute in order: the clears follow the loads above and precede the next
    // sub-block's replay; the fence keeps the compiler from reordering them.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (uint32_t i = lane * 8u; i < stage_used(p); i += kLanes * 8u) lds_store<U32x2>(stage + i, U32x2{0, 0});
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    return nxt;
  };

  if (kRows) {
    // Up to as many ids as there are workgroups, workgroup i takes id i and its eight
    // wavefronts take the sub-blocks that overlap the id's elements in turn: one round, the
    // shortest way to the few rows of a generation step.  With more ids every wavefront
    // takes ids of its own and walks a row's sub-blocks by itself, eight times as many rows
    // in flight.  Either way the next sub-block's inputs are requested a step ahead, and each
    // sub-block is written out whole, so the elements next to a row, up to a sub-block's
    // worth on either side, are decoded with it (to the same values any other decode of
    // them writes).
    const uint32_t n_entries = (uint32_t)(z.n_blocks * kSubsPerBlock + 1);
    const int64_t n_rows_total = rows.row_elements > 0 ? z.n_elements / rows.row_elements : 0;
    const bool id_per_wave = rows.n_ids > (int64_t)gridDim.x;      // uniform
    const int64_t first_id = id_per_wave ? (int64_t)blockIdx.x * kWavesPerGroup + wave : (int64_t)blockIdx.x;
    const int64_t id_stride = id_per_wave ? (int64_t)gridDim.x * kWavesPerGroup : (int64_t)gridDim.x;
    const int64_t first_sub = id_per_wave ? 0 : (int64_t)wave;
    const int64_t sub_stride = id_per_wave ? 1 : kWavesPerGroup;
    for (int64_t i = first_id; i < rows.n_ids; i += id_stride) {
      const int64_t id = rows.ids[i];                         // uniform
      if (id < 0 || id >= n_rows_total) continue;             // ids outside the matrix select nothing
      const int64_t first = id * rows.row_elements;
      const int64_t end = first + rows.row_elements;
      int64_t s = (int64_t)uniform(find_sub(subpos, n_entries, (uint32_t)first, lane)) + first_sub;
      if (s >= z.n_subs) continue;
      SubInputs in = fetch_sub<kStreaming>(codes, gaps, subpos, z, s, lane, gap_byte, vzero);
      for (;;) {
        if ((int64_t)uniform(in.base) >= end) break;          // starts past the row
        claim(in.d0, in.d1, in.d2, in.gap_raw, in.base, in.end_hint);
        const int64_t next = s + sub_stride;
        const bool more = next < z.n_subs;
        in = step(in, more, next);
        if (!more) break;
        s = next;
      }
    }
    return;
  }
  for (; sub < z.n_subs; sub += stride) {
    const int64_t next_sub = sub + stride;
    held = step(held, next_sub < z.n_subs, next_sub);
  }
}

// Launch plans.  The kernel is one body compiled for three plans; which one runs is
// decided per stream at launch time from two numbers the host knows, the number of
// sub-blocks and the elements an average sub-block produces.  Measured on MI355X
// (N(0, 0.02), Laplace, one-bit and incompressible streams of 17 M to 622 M
// elements):
//   wide     3 workgroups per CU (6 wavefronts per SIMD), 2 groups requested early,
//            plain (cacheable) loads.
//            Best when wavefronts are the scarce resource: streams whose decode is
//            bound by vector instructions (long codes, few elements per sub-block),
//            and those streams of fewer than about 38 M elements (a few rounds of
//            sub-blocks: the launch is latency-bound) whose rounds fill it well.
//   deep     2 workgroups per CU (4 per SIMD), 3 groups requested early: a typical
//            sub-block is 3 groups per lane, so the whole write-out runs on bytes
//            that are already there.  Fewer, deeper memory streams: 1 % (218 M
//            elements) to 6-8 % (622 M) faster than `wide` on weight-like streams.
//   deepest  2 workgroups per CU, 6 groups requested early, for streams of short
//            codes (a sub-block of one-bit codes is 8 groups per lane): 74 % of the
//            HBM peak on the all-zero mix against 68 % with `wide`.
// The deep plans come in a second compilation (`_short`) for streams of few
// sub-blocks per wavefront, which sets wavefront priorities by phase (see the loop),
// and `deep` in a third (`_small`) that also reads with plain loads, for the streams
// under 38 M elements that fit its rounds better than those of `wide` (a stream that
// small may still sit in the memory-side cache).  `wide` has two more compilations at
// four workgroups per CU (eight wavefronts per SIMD, all that its registers allow):
// `_full`, priorities by phase, for the streams whose sub-blocks fit one round of that
// many wavefronts, and `_dense`, priorities by rotation, for decode-bound streams.
// `portable` is `wide` with LDS addressed through its symbol (see decode_body), and
// `rows` serves df11_decode_rows.
// The register budget follows the resident wavefronts (amdgpu_waves_per_eu).
#define DF11_DECODE_KERNEL(name, prefetch, streaming, phase_priority, waves_per_simd, const_lds, slots) \
  __global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(waves_per_simd,       \
                                                                             waves_per_simd)))    \
  void name(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ sign_mantissa,         \
            const uint8_t* __restrict__ gaps, uint16_t* __restrict__ out,                         \
            const uint8_t* __restrict__ ws, const DecodeSizes z) {                                \
    decode_body<prefetch, streaming, phase_priority, const_lds, slots, (waves_per_simd < 8)>(     \
        codes, sign_mantissa, gaps, out, ws, z);                                                  \
  }
DF11_DECODE_KERNEL(decode_kernel_wide, 2, false, false, 6, true, kMainSlotsUsual)
DF11_DECODE_KERNEL(decode_kernel_deep, 3, true, false, 4, true, kMainSlotsDeep)
DF11_DECODE_KERNEL(decode_kernel_deep_short, 3, true, true, 4, true, kMainSlotsDeep)
DF11_DECODE_KERNEL(decode_kernel_deep_small, 3, false, true, 4, true, kMainSlotsDeep)
DF11_DECODE_KERNEL(decode_kernel_deepest, 6, true, false, 4, true, kMainSlotsShortCodes)
DF11_DECODE_KERNEL(decode_kernel_deepest_short, 6, true, true, 4, true, kMainSlotsShortCodes)
DF11_DECODE_KERNEL(decode_kernel_portable, 2, false, false, 6, false, kMainSlotsUsual)   // `wide`, LDS addressed through its symbol
DF11_DECODE_KERNEL(decode_kernel_wide_full, 2, false, true, 8, true, kMainSlotsFew)    // `wide` at four workgroups per CU
DF11_DECODE_KERNEL(decode_kernel_wide_dense, 2, false, false, 8, true, kMainSlotsFew)  // the same with priorities by rotation
#undef DF11_DECODE_KERNEL

// Decodes only the sub-blocks that hold given rows of the output matrix (an embedding
// looks up a few rows of a table whose stream holds them all): `wide` settings, wavefront
// priorities by phase, work taken per id (by a workgroup, or by a wavefront when the ids
// outnumber the workgroups) instead of per sub-block.
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(6, 6)))
void decode_kernel_rows(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ sign_mantissa,
                        const uint8_t* __restrict__ gaps, uint16_t* __restrict__ out,
                        const uint8_t* __restrict__ ws, const DecodeSizes z, const RowsArgs rows) {
  decode_body<2, false, true, true, kMainSlotsUsual, true, true>(codes, sign_mantissa, gaps, out, ws, z, rows);
}

typedef void (*DecodeKernel)(const uint8_t*, const uint8_t*, const uint8_t*, uint16_t*, const uint8_t*, DecodeSizes);
struct LaunchPlan {
  DecodeKernel kernel;
  int groups_per_cu;
  DecodeKernel kernel_short;   // for up to kMaxRoundsForPhasePriority sub-blocks per wavefront, or null
  const char* name;
  const char* name_short;
};
constexpr int kWideGroupsPerCu = 3;
constexpr int kDeepGroupsPerCu = 2;
constexpr int kFullGroupsPerCu = 4;   // 8 wavefronts per SIMD: every one the registers of `wide` allow
constexpr int kMinElemsPerWaveForDeep = 6144;  // output per resident wavefront of the wide plan: four typical sub-blocks
constexpr int kMinElemsPerSubForDeep = 1024;   // below: more than 4 bits per exponent, decode-bound
constexpr int kMinElemsPerSubForManyLookups = 480;   // below: codes so long that seven lookups cover a chunk
constexpr int kMinElemsPerSubForDeepest = 2048;   // two bits per code and fewer: sparse weights, one-bit streams
// Up to this many sub-blocks per wavefront, the deep plans set wavefront priorities by
// phase (4096x14336 to 100 M elements: 2-7 % faster than by turn; equal at 120 M to
// 142 M; 0.5 % slower at 218 M, 5 % at 622 M; 9 % slower under the wide plan on a
// decode-bound stream).
constexpr int kMaxRoundsForPhasePriority = 16;
constexpr int64_t kMaxInputBytesForPlainLoads = 40 << 20;   // about 30 M weight-like elements

const LaunchPlan kWide{decode_kernel_wide, kWideGroupsPerCu, nullptr, "wide", nullptr};
const LaunchPlan kWideFull{decode_kernel_wide_full, kFullGroupsPerCu, nullptr, "wide/full", nullptr};
const LaunchPlan kWideDense{decode_kernel_wide_dense, kFullGroupsPerCu, nullptr, "wide/dense", nullptr};
const LaunchPlan kDeep{decode_kernel_deep, kDeepGroupsPerCu, decode_kernel_deep_short, "deep", "deep/short"};
const LaunchPlan kDeepSmall{decode_kernel_deep_small, kDeepGroupsPerCu, decode_kernel_deep_small, "deep/small",
                            "deep/small"};
const LaunchPlan kDeepest{decode_kernel_deepest, kDeepGroupsPerCu, decode_kernel_deepest_short, "deepest",
                          "deepest/short"};
const LaunchPlan kPortable{decode_kernel_portable, kWideGroupsPerCu, nullptr, "portable", nullptr};

// `pinned` is one of DF11_PLAN_*: anything but a plan's number leaves the choice to the rule.
LaunchPlan plan_launch(int64_t n_subs, int64_t n_elements, int cus, int pinned = DF11_PLAN_AUTO) {
  switch (pinned) {
    case DF11_PLAN_WIDE: return kWide;
    case DF11_PLAN_DEEP: return kDeep;
    case DF11_PLAN_DEEPEST: return kDeepest;
    case DF11_PLAN_PORTABLE: return kPortable;
    default: break;
  }
  const int64_t wide_waves = (int64_t)cus * kWideGroupsPerCu * kWavesPerGroup;
  const int64_t deep_waves = (int64_t)cus * kDeepGroupsPerCu * kWavesPerGroup;
  const int64_t elems_per_sub = n_subs ? n_elements / n_subs : 0;
  // Decode-bound streams.  With more than 8.5 bits per code on average (fewer than 480
  // elements per sub-block) seven lookups cover a chunk, and the stream gains from every
  // wavefront the registers allow (incompressible exponents, 8 M to 622 M elements: 2.5-5 %
  // faster at four workgroups per CU than at three).  Codes of 5.5 to 8.5 bits take eight to
  // ten lookups per chunk, which only the compilations with more register slots hold.
  if (elems_per_sub < kMinElemsPerSubForManyLookups) return kWideDense;
  if (elems_per_sub < kMinElemsPerSubForDeep) return kWide;
  if (n_elements < kMinElemsPerWaveForDeep * wide_waves) {
    // A few rounds of sub-blocks: the launch is bound by latency, and what counts is how
    // the sub-blocks fill the rounds of the wavefronts a plan keeps resident (W = 6144 on
    // 256 CUs for wide, 2/3 W for deep, 4/3 W for wide/full).  Under the wide plan such a
    // launch takes as long as its rounds, full or not; under the deep plan it grows more
    // evenly with the stream.  Measured on N(0, 0.02) streams of 2 M to 38 M elements read
    // from HBM (time per launch, best plan against the next):
    //   up to one round of deep               deep/small  (4 M elements: 7.8 against 8.4 us)
    //   up to one round of wide/full          wide/full   (8 M: 9.6 against 9.9 us; 10 M: 12.0 against
    //                                                      13.4 us, 12 M: 12.6 against 14.6 us: one
    //                                                      round instead of a full round of wide
    //                                                      and a nearly empty one)
    //   up to two rounds of wide              wide        (13 M: 14.7 against 16.9 us, 16.8 M: 17.1
    //                                                      against 17.6 us)
    //   beyond                                deep        (20 M: 19.3 against 20.9 us, 28 M: 24.4
    //                                                      against 26.0 us)
    // Short-code streams stay wide.
    if (elems_per_sub >= kMinElemsPerSubForDeepest) return kWide;
    const int64_t full_waves = (int64_t)cus * kFullGroupsPerCu * kWavesPerGroup;
    if (n_subs > deep_waves && n_subs <= 2 * wide_waves) return n_subs <= full_waves ? kWideFull : kWide;
    // Plain loads pay when the stream may still be in the memory-side cache and cost 1-5 %
    // when it comes from HBM, more the larger it is.
    const int64_t input_bytes = n_subs * kSubBytes + n_elements;
    return input_bytes < kMaxInputBytesForPlainLoads ? kDeepSmall : kDeep;
  }
  if (elems_per_sub < kMinElemsPerSubForDeepest) return kDeep;
  return kDeepest;
}

bool few_rounds(int64_t n_subs, int64_t grid) {
  return n_subs <= (int64_t)kMaxRoundsForPhasePriority * grid * kWavesPerGroup;
}

struct DeviceInfo {
  int cus = 0;
  bool constant_lds_base = false;   // the kernels that address LDS from a constant may run
  bool ok = false;
};

int device_info(DeviceInfo& info) {
  thread_local DeviceInfo cache[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e);
  if (dev < 0 || dev >= 64) return DF11_ERR_UNSUPPORTED;
  if (!cache[dev].ok) {
    int cus = 0;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return hip_fail(e);
    // the decode kernels address their LDS from a constant base, which holds only
    // as long as they have no static LDS of their own; if one of them has, every
    // stream runs the compilation that takes the base from the symbol instead
    bool constant_base = true;
    for (const void* k : {reinterpret_cast<const void*>(decode_kernel_wide), reinterpret_cast<const void*>(decode_kernel_deep),
                          reinterpret_cast<const void*>(decode_kernel_deep_short),
                          reinterpret_cast<const void*>(decode_kernel_deep_small),
                          reinterpret_cast<const void*>(decode_kernel_deepest),
                          reinterpret_cast<const void*>(decode_kernel_deepest_short),
                          reinterpret_cast<const void*>(decode_kernel_wide_full),
                          reinterpret_cast<const void*>(decode_kernel_wide_dense),
                          reinterpret_cast<const void*>(decode_kernel_rows)}) {
      hipFuncAttributes attr;
      e = hipFuncGetAttributes(&attr, k);
      if (e != hipSuccess) return hip_fail(e);
      if (attr.sharedSizeBytes != 0) constant_base = false;
    }
    cache[dev].constant_lds_base = constant_base;
    cache[dev].cus = cus;
    cache[dev].ok = true;
  }
  info = cache[dev];
  return DF11_OK;
}

constexpr int kLdsPerCu = 160 * 1024;

// Workgroups of lds_bytes each that fit a CU, at most `wanted`.
int groups_per_cu(size_t lds_bytes, int wanted) {
  int n = (int)(kLdsPerCu / lds_bytes);
  if (n > wanted) n = wanted;
  return n < 1 ? 1 : n;
}

// Enqueues the two load-time kernels that fill `ws` for one stream.
int enqueue_prepare(const uint8_t* luts, const uint8_t* encoded_exponent, const uint32_t* output_positions,
                    const uint8_t* gaps, int32_t n_luts, int64_t n_bytes, int64_t n_elements, uint8_t* ws,
                    const DeviceInfo& info, hipStream_t s) {
  const int64_t n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  hipLaunchKernelGGL(build_tables_kernel, dim3(kTableEntries / 256), dim3(256), 0, s, luts, (int)n_luts,
                     ws, (uint32_t)n_blocks);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  if (n_blocks > 0) {
    IndexArgs a;
    a.codes = encoded_exponent;
    a.positions = output_positions;
    a.gaps = gaps;
    a.ws = ws;
    a.n_bytes = n_bytes;
    a.n_elements = n_elements;
    a.n_blocks = n_blocks;
    a.n_luts = n_luts;
    a.codes_aligned = (reinterpret_cast<uintptr_t>(encoded_exponent) & 7) == 0;
    const size_t lds_bytes = (size_t)kTablesBytes + 64;
    int64_t grid = (int64_t)info.cus * groups_per_cu(lds_bytes, kWideGroupsPerCu);
    if (grid > n_blocks) grid = n_blocks;
    hipLaunchKernelGGL(index_kernel, dim3((unsigned)grid), dim3(kThreads), lds_bytes, s, a);
    e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
  }
  return DF11_OK;
}

// Sizes and alignment facts of a stream as the decode kernels take them.
DecodeSizes decode_sizes(const uint8_t* encoded_exponent, const uint8_t* sign_mantissa, const uint16_t* outputs,
                         int32_t n_luts, int64_t n_bytes, int64_t n_elements, int32_t max_elems_per_subblock) {
  if (max_elems_per_subblock <= 0 || max_elems_per_subblock > kMaxElemsPerSub)
    max_elems_per_subblock = kMaxElemsPerSub;
  DecodeSizes z;
  z.n_bytes = n_bytes;
  z.n_elements = n_elements;
  z.n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  z.n_subs = (n_bytes + kSubBytes - 1) / kSubBytes;
  z.n_luts = n_luts;
  z.stage_cap = stage_capacity(max_elems_per_subblock);
  z.codes_aligned = (reinterpret_cast<uintptr_t>(encoded_exponent) & 7) == 0;
  z.vec_ok = (reinterpret_cast<uintptr_t>(sign_mantissa) & 7) == 0 &&
             (reinterpret_cast<uintptr_t>(outputs) & 15) == 0;
  return z;
}

// LDS of one workgroup: tables, the fused LUT rows that exist, one staging area per wavefront.
size_t decode_lds_bytes(const DecodeSizes& z) {
  const int n_rows = z.n_luts - 1 < kMaxDecodeRows ? z.n_luts - 1 : kMaxDecodeRows;
  return (size_t)kLdsSkip + (size_t)tables_bytes(n_rows) + (size_t)kWavesPerGroup * (size_t)z.stage_cap;
}

// Enqueues the decode of one stream whose workspace `ws` is (or will be, in
// stream order) filled.
int enqueue_decode(const uint8_t* luts, const uint8_t* encoded_exponent, const uint8_t* sign_mantissa,
                   const uint8_t* gaps, uint16_t* outputs, int32_t n_luts, int64_t n_bytes,
                   int64_t n_elements, const uint8_t* ws, int32_t max_elems_per_subblock,
                   const DeviceInfo& info, hipStream_t s, int pinned_plan = DF11_PLAN_AUTO) {
  const DecodeSizes z = decode_sizes(encoded_exponent, sign_mantissa, outputs, n_luts, n_bytes, n_elements,
                                     max_elems_per_subblock);
  const size_t lds_bytes = decode_lds_bytes(z);
  const LaunchPlan plan = plan_launch(z.n_subs, n_elements, info.cus,
                                      info.constant_lds_base ? pinned_plan : DF11_PLAN_PORTABLE);
  int64_t grid = (int64_t)info.cus * groups_per_cu(lds_bytes, plan.groups_per_cu);
  const int64_t needed = (z.n_subs + kWavesPerGroup - 1) / kWavesPerGroup;
  if (grid > needed) grid = needed;
  const DecodeKernel kernel = few_rounds(z.n_subs, grid) && plan.kernel_short ? plan.kernel_short : plan.kernel;

  (void)luts;   // read by df11_prepare only: the decode finds them fused in the workspace
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kThreads), lds_bytes, s,
                     encoded_exponent, sign_mantissa, gaps, outputs, ws, z);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DF11_OK : hip_fail(e);
}

// ---------------------------------------------------------------------------
// Library-owned workspace for callers that cannot allocate device memory.
// `scratch` is a host-side stand-in for the device array: host code never uses
// the name as an address, only the per-device pointer that
// hipGetSymbolAddress returns (each GPU holds its own copy of the array).
// ---------------------------------------------------------------------------
static __device__ __align__(256) uint8_t scratch[DF11_STATIC_WORKSPACE_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint8_t* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, looked up once per device.
int scratch_of_current_device(uint8_t** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e);
  if (dev < 0 || dev >= kMaxDevices) return DF11_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e);
    if (!p) return DF11_ERR_HIP;
    g_scratch_ptr[dev] = static_cast<uint8_t*>(p);
  }
  *out = g_scratch_ptr[dev];
  return DF11_OK;
}

}  // namespace

extern "C" {

int df11_version(void) { return 5; }

const char* df11_error_string(int code) {
  switch (code) {
    case DF11_OK: return "ok";
    case DF11_ERR_INVALID_ARGUMENT: return "invalid argument";
    case DF11_ERR_UNSUPPORTED: return "unsupported configuration";
    case DF11_ERR_HIP: return "HIP runtime error";
    case DF11_ERR_CAPACITY: return "buffer too small or fixed capacity exceeded";
    case DF11_ERR_FORMAT: return "code not expressible in the DF11 LUT layout";
    default: return "unknown error";
  }
}

const char* df11_last_hip_error(void) { return hipGetErrorString(g_last_hip); }

size_t df11_workspace_bytes(int64_t n_bytes) {
  if (n_bytes < 0) return 0;
  return (size_t)workspace_bytes((n_bytes + kBlockBytes - 1) / kBlockBytes);
}

int df11_prepare(const uint8_t* luts, const uint8_t* encoded_exponent, const uint32_t* output_positions,
                 const uint8_t* gaps, int32_t n_luts, int64_t n_bytes, int64_t n_elements,
                 void* workspace, int32_t* max_elems_per_subblock, void* stream) {
  if (n_bytes < 0 || n_elements < 0 || n_luts < 2 || !luts || !workspace) return DF11_ERR_INVALID_ARGUMENT;
  if (n_elements >= ((int64_t)1 << 32)) return DF11_ERR_UNSUPPORTED;   // positions are u32
  if (n_bytes > 0 && (!encoded_exponent || !output_positions || !gaps)) return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(workspace) & 15) || (reinterpret_cast<uintptr_t>(output_positions) & 3))
    return DF11_ERR_INVALID_ARGUMENT;
  DeviceInfo info;
  if (int rc = device_info(info)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  if (n_blocks >= ((int64_t)1 << 28)) return DF11_ERR_UNSUPPORTED;
  uint8_t* ws = static_cast<uint8_t*>(workspace);

  if (int rc = enqueue_prepare(luts, encoded_exponent, output_positions, gaps, n_luts, n_bytes, n_elements, ws,
                               info, s))
    return rc;
  hipError_t e = hipSuccess;
  if (max_elems_per_subblock) {
    WorkspaceHeader h;
    e = hipMemcpyAsync(&h, ws, sizeof h, hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return hip_fail(e);
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(e);
    *max_elems_per_subblock = (int32_t)h.max_sub_elems;
  }
  return DF11_OK;
}

const char* df11_launch_plan_name(int64_t n_bytes, int64_t n_elements, int32_t compute_units) {
  if (n_bytes <= 0 || n_elements <= 0 || compute_units <= 0) return "";
  const int64_t n_subs = (n_bytes + kSubBytes - 1) / kSubBytes;
  const LaunchPlan plan = plan_launch(n_subs, n_elements, compute_units);
  int64_t grid = (int64_t)compute_units * plan.groups_per_cu;
  const int64_t needed = (n_subs + kWavesPerGroup - 1) / kWavesPerGroup;
  if (grid > needed) grid = needed;
  return few_rounds(n_subs, grid) && plan.kernel_short ? plan.name_short : plan.name;
}

namespace {
int checked_decode(const uint8_t* luts, const uint8_t* encoded_exponent, const uint8_t* sign_mantissa,
                   const uint8_t* gaps, uint16_t* outputs, int32_t n_luts, int64_t n_bytes, int64_t n_elements,
                   const void* workspace, int32_t max_elems_per_subblock, void* stream, int pinned_plan) {
  if (n_bytes < 0 || n_elements < 0 || n_luts < 2) return DF11_ERR_INVALID_ARGUMENT;
  if (n_bytes == 0 || n_elements == 0) return DF11_OK;
  if (!luts || !encoded_exponent || !sign_mantissa || !gaps || !outputs || !workspace)
    return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(workspace) & 15) || (reinterpret_cast<uintptr_t>(outputs) & 1))
    return DF11_ERR_INVALID_ARGUMENT;
  if (n_elements >= ((int64_t)1 << 32)) return DF11_ERR_UNSUPPORTED;   // positions are u32
  DeviceInfo info;
  if (int rc = device_info(info)) return rc;
  return enqueue_decode(luts, encoded_exponent, sign_mantissa, gaps, outputs, n_luts, n_bytes, n_elements,
                        static_cast<const uint8_t*>(workspace), max_elems_per_subblock, info,
                        static_cast<hipStream_t>(stream), pinned_plan);
}
}  // namespace

int df11_decode(const uint8_t* luts, const uint8_t* encoded_exponent, const uint8_t* sign_mantissa,
                const uint32_t* output_positions, const uint8_t* gaps, uint16_t* outputs,
                int32_t n_luts, int64_t n_bytes, int64_t n_elements, const void* workspace,
                int32_t max_elems_per_subblock, void* stream) {
  (void)output_positions;   // superseded by the sub-block positions in the workspace
  return checked_decode(luts, encoded_exponent, sign_mantissa, gaps, outputs, n_luts, n_bytes, n_elements, workspace,
                        max_elems_per_subblock, stream, DF11_PLAN_AUTO);
}

int df11_decode_with_plan(const uint8_t* luts, const uint8_t* encoded_exponent, const uint8_t* sign_mantissa,
                          const uint32_t* output_positions, const uint8_t* gaps, uint16_t* outputs,
                          int32_t n_luts, int64_t n_bytes, int64_t n_elements, const void* workspace,
                          int32_t max_elems_per_subblock, void* stream, int32_t plan) {
  (void)output_positions;
  if (plan < DF11_PLAN_AUTO || plan > DF11_PLAN_PORTABLE) return DF11_ERR_INVALID_ARGUMENT;
  return checked_decode(luts, encoded_exponent, sign_mantissa, gaps, outputs, n_luts, n_bytes, n_elements, workspace,
                        max_elems_per_subblock, stream, plan);
}

int df11_decode_rows(const uint8_t* luts, const uint8_t* encoded_exponent, const uint8_t* sign_mantissa,
                     const uint32_t* output_positions, const uint8_t* gaps, uint16_t* outputs,
                     int32_t n_luts, int64_t n_bytes, int64_t n_elements, const void* workspace,
                     int32_t max_elems_per_subblock, void* stream, const int64_t* row_ids, int64_t n_ids,
                     int64_t row_elements) {
  (void)output_positions;
  if (n_bytes < 0 || n_elements < 0 || n_luts < 2 || n_ids < 0 || row_elements <= 0) return DF11_ERR_INVALID_ARGUMENT;
  if (n_bytes == 0 || n_elements == 0 || n_ids == 0) return DF11_OK;
  if (!luts || !encoded_exponent || !sign_mantissa || !gaps || !outputs || !workspace || !row_ids)
    return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(workspace) & 15) || (reinterpret_cast<uintptr_t>(outputs) & 1) ||
      (reinterpret_cast<uintptr_t>(row_ids) & 7))
    return DF11_ERR_INVALID_ARGUMENT;
  if (n_elements >= ((int64_t)1 << 32)) return DF11_ERR_UNSUPPORTED;   // positions are u32
  DeviceInfo info;
  if (int rc = device_info(info)) return rc;
  if (!info.constant_lds_base) return DF11_ERR_UNSUPPORTED;   // callers decode the whole stream instead
  const DecodeSizes z = decode_sizes(encoded_exponent, sign_mantissa, outputs, n_luts, n_bytes, n_elements,
                                     max_elems_per_subblock);
  const size_t lds_bytes = decode_lds_bytes(z);
  int64_t grid = (int64_t)info.cus * groups_per_cu(lds_bytes, kWideGroupsPerCu);
  if (grid > n_ids) grid = n_ids;
  RowsArgs rows;
  rows.ids = row_ids;
  rows.n_ids = n_ids;
  rows.row_elements = row_elements;
  hipLaunchKernelGGL(decode_kernel_rows, dim3((unsigned)grid), dim3(kThreads), lds_bytes,
                     static_cast<hipStream_t>(stream), encoded_exponent, sign_mantissa, gaps, outputs,
                     static_cast<const uint8_t*>(workspace), z, rows);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DF11_OK : hip_fail(e);
}

int df11_decode_static_workspace(const uint8_t* luts, const uint8_t* encoded_exponent,
                                 const uint8_t* sign_mantissa, const uint32_t* output_positions,
                                 const uint8_t* gaps, uint16_t* outputs, int32_t n_luts, int64_t n_bytes,
                                 int64_t n_elements, int32_t max_elems_per_subblock, void* stream) {
  if (n_bytes < 0 || n_elements < 0 || n_luts < 2) return DF11_ERR_INVALID_ARGUMENT;
  if (n_bytes == 0 || n_elements == 0) return DF11_OK;
  if (!luts || !encoded_exponent || !sign_mantissa || !output_positions || !gaps || !outputs)
    return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(output_positions) & 3) || (reinterpret_cast<uintptr_t>(outputs) & 1))
    return DF11_ERR_INVALID_ARGUMENT;
  if (n_elements >= ((int64_t)1 << 32)) return DF11_ERR_UNSUPPORTED;   // positions are u32
  // the stream's workspace must fit the library's static array
  if (n_bytes > (int64_t)DF11_STATIC_MAX_STREAM_BYTES) return DF11_ERR_CAPACITY;
  const int64_t n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  if (workspace_bytes(n_blocks) > (int64_t)DF11_STATIC_WORKSPACE_BYTES) return DF11_ERR_CAPACITY;
  DeviceInfo info;
  if (int rc = device_info(info)) return rc;
  uint8_t* ws = nullptr;
  if (int rc = scratch_of_current_device(&ws)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // The header word that accumulates a maximum is reset by build_tables_kernel
  // itself; tables and positions are overwritten in full for this stream's size.
  if (int rc = enqueue_prepare(luts, encoded_exponent, output_positions, gaps, n_luts, n_bytes, n_elements, ws,
                               info, s))
    return rc;
  return enqueue_decode(luts, encoded_exponent, sign_mantissa, gaps, outputs, n_luts, n_bytes, n_elements, ws,
                        max_elems_per_subblock, info, s);
}

}  // extern "C"
