// gfx950 kernels and C-ABI for DF11 stream decode.
//
// One workgroup of 512 threads (8 wavefronts of 64) handles one 4096-byte
// bitstream block at a time and walks the grid persistently, so the derived
// tables are copied into LDS once per workgroup rather than once per block.
// Per block:
//   1. every thread takes its 8-byte chunk (+4 bytes of look-ahead) and 5-bit gap
//      (fetched one block ahead) and counts the codes starting in the chunk with
//      the four-symbol table in LDS;
//   2. exclusive prefix sum of the 512 counts: DPP scan inside each wavefront,
//      eight wavefront totals combined through LDS;
//   3. every thread decodes its codes again and stores the symbols of each lookup
//      with one unaligned 32-bit LDS store into a staging area laid out in output
//      order;
//   4. the workgroup streams the staging area out: 16 exponent bytes (LDS) + 16
//      sign|mantissa bytes (global, coalesced, requested before step 1) -> two
//      16-byte BF16 stores per lane.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/df11.h"
#include "df11_core.h"

namespace {

using namespace df11;

thread_local hipError_t g_last_hip = hipSuccess;

inline int hip_fail(hipError_t e) {
  g_last_hip = e;
  return DF11_ERR_HIP;
}

// ---------------------------------------------------------------------------
// Table builder: one thread per table index.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void build_tables_kernel(const uint8_t* __restrict__ luts,
                                                           int n_luts, uint8_t* __restrict__ tables) {
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (uint32_t)kTableEntries) return;
  // The length row is the last row of `luts`; decode rows beyond the 17 a
  // pointer can name are unreachable.  Present both as one contiguous view by
  // staging into LDS: rows [0, n_rows) then the length row.
  __shared__ uint8_t rows[(kMaxDecodeRows + 1) * 256];
  const int n_rows = min(n_luts - 1, kMaxDecodeRows);
  for (int i = threadIdx.x; i < n_rows * 256; i += blockDim.x) rows[i] = luts[i];
  for (int i = threadIdx.x; i < 256; i += blockDim.x)
    rows[n_rows * 256 + i] = luts[(n_luts - 1) * 256 + i];
  __syncthreads();
  Luts l{rows, n_rows};
  uint32_t syms, meta;
  make_dec_entry(l, idx, syms, meta);
  reinterpret_cast<uint2*>(tables + kDecOffset)[idx] = make_uint2(syms, meta);
  tables[kCntTailOffset + idx] = make_cnt_tail_entry(l, idx);
}

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

// ---------------------------------------------------------------------------
// Decode kernel.
// LDS layout (dynamic): tables | byte LUT rows + length row | wave sums | stage
// ---------------------------------------------------------------------------
struct DecodeArgs {
  const uint8_t* luts;
  const uint8_t* codes;
  const uint8_t* sign_mantissa;
  const uint32_t* positions;
  const uint8_t* gaps;
  uint16_t* out;
  const uint8_t* tables;
  int64_t n_bytes;
  int64_t n_elements;
  int64_t n_blocks;
  int32_t n_luts;
  int32_t stage_cap;      // bytes of staging, multiple of 16
  int32_t codes_aligned;  // codes pointer is 8-byte aligned
  int32_t vec_ok;         // sign_mantissa and out both 16-byte aligned
};

__global__ __launch_bounds__(kThreads) void decode_kernel(const DecodeArgs a) {
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  const int n_rows = min(a.n_luts - 1, kMaxDecodeRows);
  uint8_t* lds_tables = lds;
  uint8_t* lds_rows = lds + kTablesBytes;
  uint32_t* wave_sums = reinterpret_cast<uint32_t*>(lds_rows + (kMaxDecodeRows + 1) * 256);
  uint8_t* stage = reinterpret_cast<uint8_t*>(wave_sums + 16);

  // Tables and byte LUTs into LDS, 16 bytes per lane per step.
  {
    const uint4* src = reinterpret_cast<const uint4*>(a.tables);
    uint4* dst = reinterpret_cast<uint4*>(lds_tables);
    for (int i = tid; i < kTablesBytes / 16; i += kThreads) dst[i] = src[i];
    for (int i = tid; i < n_rows * 256; i += kThreads) lds_rows[i] = a.luts[i];
    if (tid < 256) lds_rows[n_rows * 256 + tid] = a.luts[(int64_t)(a.n_luts - 1) * 256 + tid];
  }
  __syncthreads();

  const Tables t{lds_tables + kDecOffset, lds_tables + kCntTailOffset};
  const Luts l{lds_rows, n_rows};
  const int64_t n_gap_bytes = a.n_blocks * kGapBytesPerBlock;
  const bool vec_ok = a.vec_ok != 0;

  int64_t blk = blockIdx.x;
  Chunk c = fetch_chunk(a.codes, a.n_bytes, blk * kThreads + tid, a.codes_aligned != 0);
  uint32_t gap = gap_of(a.gaps, blk * kThreads + tid, n_gap_bytes);

  for (; blk < a.n_blocks; blk += gridDim.x) {
    // ---- requests whose latency the two decode passes hide: the next block's
    // chunk and gap, and this block's sign|mantissa bytes for the write-out
    const int64_t next_blk = blk + gridDim.x;
    Chunk c_next{0, 0, 0};
    uint32_t gap_next = 0;
    if (next_blk < a.n_blocks) {
      c_next = fetch_chunk(a.codes, a.n_bytes, next_blk * kThreads + tid, a.codes_aligned != 0);
      gap_next = gap_of(a.gaps, next_blk * kThreads + tid, n_gap_bytes);
    }
    const int64_t base = (int64_t)a.positions[blk];
    const int64_t a0 = base & ~(int64_t)(kGroup - 1);
    U32x4 m0{0, 0, 0, 0}, m1{0, 0, 0, 0};
    if (vec_ok) {
      const int64_t i0 = a0 + (int64_t)tid * kGroup, i1 = i0 + (int64_t)kThreads * kGroup;
      if (i0 + kGroup <= a.n_elements) m0 = load_as<U32x4>(a.sign_mantissa + i0);
      if (i1 + kGroup <= a.n_elements) m1 = load_as<U32x4>(a.sign_mantissa + i1);
    }

    // ---- pass 1: how many codes start in my chunk
    const uint32_t count = count_chunk(t, l, c.hi, c.lo, c.next, gap);

    // ---- exclusive prefix over the workgroup
    const uint32_t incl = wave_inclusive_scan(count);
    if (lane == 63) wave_sums[wave] = incl;
    __syncthreads();
    uint32_t wave_base = 0, total = 0;
#pragma unroll
    for (int wv = 0; wv < kThreads / 64; ++wv) {
      const uint32_t s = wave_sums[wv];
      if (wv < wave) wave_base += s;
      total += s;
    }
    const uint32_t excl = wave_base + incl - count;

    // ---- pass 2: decode into the staging area, in output order
    const BlockPlan p = plan_block(base, total, a.n_elements, a.stage_cap);
    emit_chunk(t, l, c.hi, c.lo, c.next, gap, thread_quota(excl, count, p.n_out),
               stage + p.phase + excl);
    __syncthreads();

    // ---- stream out, 16 elements per lane per step.  No barrier is needed after
    // this: the next block's staging writes come after its prefix-sum barrier,
    // which every wavefront reaches only when it is done reading here.
    const uint32_t n_groups = n_groups_of(p);
    for (uint32_t g = tid; g < n_groups; g += kThreads) {
      if (vec_ok && group_is_full(g, p)) {
        U32x4 m;
        if (g == (uint32_t)tid) m = m0;
        else if (g == (uint32_t)(tid + kThreads)) m = m1;
        else m = load_as<U32x4>(a.sign_mantissa + p.a0 + (int64_t)g * kGroup);
        stream_group_full(g, p, stage, m, a.out);
      } else {
        stream_group_ragged(g, p, stage, a.sign_mantissa, a.out);
      }
    }
    c = c_next;
    gap = gap_next;
  }
}

// Plain streaming copy, 16 bytes per lane: the known-traffic kernel against
// which hardware byte counters are calibrated.
__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src,
                                                   uint4* __restrict__ dst, int64_t n_vec) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

struct DeviceInfo {
  int cus = 0;
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
    cache[dev].cus = cus;
    cache[dev].ok = true;
  }
  info = cache[dev];
  return DF11_OK;
}

constexpr int kFixedLds = kTablesBytes + (kMaxDecodeRows + 1) * 256 + 16 * 4;

}  // namespace

extern "C" {

int df11_version(void) { return 1; }

const char* df11_error_string(int code) {
  switch (code) {
    case DF11_OK: return "ok";
    case DF11_ERR_INVALID_ARGUMENT: return "invalid argument";
    case DF11_ERR_UNSUPPORTED: return "unsupported configuration";
    case DF11_ERR_HIP: return "HIP runtime error";
    case DF11_ERR_CAPACITY: return "output buffer too small";
    case DF11_ERR_FORMAT: return "code not expressible in the DF11 LUT layout";
    default: return "unknown error";
  }
}

const char* df11_last_hip_error(void) { return hipGetErrorString(g_last_hip); }

size_t df11_tables_bytes(void) { return kTablesBytes; }

int df11_build_tables(const uint8_t* luts, int32_t n_luts, void* tables, void* stream) {
  if (!luts || !tables || n_luts < 2) return DF11_ERR_INVALID_ARGUMENT;
  if (reinterpret_cast<uintptr_t>(tables) & 15) return DF11_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(build_tables_kernel, dim3(kTableEntries / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), luts, (int)n_luts,
                     static_cast<uint8_t*>(tables));
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DF11_OK : hip_fail(e);
}

int df11_calibration_copy(const void* src, void* dst, int64_t n_bytes, void* stream) {
  if (!src || !dst || n_bytes <= 0 || (n_bytes & 15)) return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15)
    return DF11_ERR_INVALID_ARGUMENT;
  DeviceInfo info;
  if (int rc = device_info(info)) return rc;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)(info.cus * 8)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(src),
                     static_cast<uint4*>(dst), n_bytes / 16);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DF11_OK : hip_fail(e);
}

int df11_decode(const uint8_t* luts, const uint8_t* encoded_exponent, const uint8_t* sign_mantissa,
                const uint32_t* output_positions, const uint8_t* gaps, uint16_t* outputs,
                int32_t n_luts, int64_t n_bytes, int64_t n_elements, int32_t max_elems_per_block,
                const void* tables, void* stream) {
  if (n_bytes < 0 || n_elements < 0 || n_luts < 2) return DF11_ERR_INVALID_ARGUMENT;
  if (n_bytes == 0 || n_elements == 0) return DF11_OK;
  if (!luts || !encoded_exponent || !sign_mantissa || !output_positions || !gaps || !outputs || !tables)
    return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(tables) & 15) || (reinterpret_cast<uintptr_t>(outputs) & 1) ||
      (reinterpret_cast<uintptr_t>(output_positions) & 3))
    return DF11_ERR_INVALID_ARGUMENT;
  if (max_elems_per_block <= 0 || max_elems_per_block > kMaxElemsPerBlock)
    max_elems_per_block = kMaxElemsPerBlock;

  DeviceInfo info;
  if (int rc = device_info(info)) return rc;

  DecodeArgs a;
  a.luts = luts;
  a.codes = encoded_exponent;
  a.sign_mantissa = sign_mantissa;
  a.positions = output_positions;
  a.gaps = gaps;
  a.out = outputs;
  a.tables = static_cast<const uint8_t*>(tables);
  a.n_bytes = n_bytes;
  a.n_elements = n_elements;
  a.n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  a.n_luts = n_luts;
  a.stage_cap = ((max_elems_per_block + kGroup + 15) / 16) * 16;   // + up to 15 elements of output phase
  a.codes_aligned = (reinterpret_cast<uintptr_t>(encoded_exponent) & 7) == 0;
  a.vec_ok = (reinterpret_cast<uintptr_t>(sign_mantissa) & 15) == 0 &&
             (reinterpret_cast<uintptr_t>(outputs) & 15) == 0;

  const size_t lds_bytes = (size_t)kFixedLds + (size_t)a.stage_cap;
  int wgs_per_cu = (int)((160 * 1024) / lds_bytes);
  if (wgs_per_cu > 4) wgs_per_cu = 4;     // 2048 threads per CU
  if (wgs_per_cu < 1) wgs_per_cu = 1;
  int64_t grid = (int64_t)info.cus * wgs_per_cu;
  if (grid > a.n_blocks) grid = a.n_blocks;

  hipLaunchKernelGGL(decode_kernel, dim3((unsigned)grid), dim3(kThreads), lds_bytes,
                     static_cast<hipStream_t>(stream), a);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DF11_OK : hip_fail(e);
}

}  // extern "C"
