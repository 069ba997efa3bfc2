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
//   2. counts the codes starting in each lane's chunk (four-symbol table in LDS);
//   3. turns the 64 counts into exclusive offsets with a DPP scan;
//   4. decodes again, storing the symbols of each lookup with one unaligned
//      32-bit store into its private LDS staging area, in output order;
//   5. streams the staging area out: 8 exponent bytes (LDS) + 8 sign|mantissa
//      bytes -> one 16-byte BF16 store per lane, contiguous across the wavefront.
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

constexpr int kWavesPerGroup = kThreads / kLanes;   // 8

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

__device__ __forceinline__ uint32_t wave_total(uint32_t inclusive) {
  return (uint32_t)__builtin_amdgcn_readlane((int)inclusive, 63);
}

// Copies the byte LUT rows a pointer can reach, then the length row, into LDS.
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
  if (idx < sizeof(WorkspaceHeader) / 4) {
    uint32_t v = 0;
    if (idx == 0) v = kWorkspaceMagic;
    if (idx == 1) v = n_blocks;
    reinterpret_cast<uint32_t*>(ws)[idx] = v;   // max_sub_elems starts at 0
  }
}

// ---------------------------------------------------------------------------
// Prepare, step 2: where each sub-block's output starts.  One workgroup per
// 4096-byte block at a time: count per lane, totals per wavefront, offsets from
// the block's own output position.
// ---------------------------------------------------------------------------
struct IndexArgs {
  const uint8_t* luts;
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
  uint8_t* lds_tables = lds;
  uint8_t* lds_rows = lds + kTablesBytes;
  uint32_t* wave_sums = reinterpret_cast<uint32_t*>(lds_rows + (kMaxDecodeRows + 1) * 256);
  {
    const uint4* src = reinterpret_cast<const uint4*>(a.ws + kWsTablesOffset);
    uint4* dst = reinterpret_cast<uint4*>(lds_tables);
    for (int i = tid; i < kTablesBytes / 16; i += kThreads) dst[i] = src[i];
    stage_rows(a.luts, a.n_luts, n_rows, lds_rows, tid, kThreads);
  }
  __syncthreads();
  const Tables t{lds_tables + kDecOffset, lds_tables + kCntTailOffset};
  const Luts l{lds_rows, n_rows};
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
// LDS layout (dynamic): tables | byte LUT rows + length row | 8 staging areas
// ---------------------------------------------------------------------------
struct DecodeArgs {
  const uint8_t* luts;
  const uint8_t* codes;
  const uint8_t* sign_mantissa;
  const uint8_t* gaps;
  uint16_t* out;
  const uint8_t* ws;
  int64_t n_bytes;
  int64_t n_elements;
  int64_t n_blocks;
  int64_t n_subs;         // sub-blocks that hold stream bytes: ceil(n_bytes / 512)
  int32_t n_luts;
  int32_t stage_cap;      // bytes of staging per wavefront, multiple of 16
  int32_t codes_aligned;  // codes pointer is 8-byte aligned
  int32_t vec_ok;         // sign_mantissa 8-byte aligned and out 16-byte aligned
};

constexpr int kPrefetchGroups = 3;   // body groups per lane whose sign|mantissa bytes are requested early

struct SubInputs {
  Chunk c;
  uint32_t gap;
  uint32_t base;       // first output element
  uint32_t end_hint;   // first output element of the next sub-block
};

__device__ __forceinline__ SubInputs fetch_sub(const DecodeArgs& a, const uint32_t* subpos, int64_t sub,
                                               int lane, int64_t n_gap_bytes) {
  SubInputs in;
  const int64_t gid = sub * kLanes + lane;
  in.c = fetch_chunk(a.codes, a.n_bytes, gid, a.codes_aligned != 0);
  in.gap = gap_of(a.gaps, gid, n_gap_bytes);
  in.base = subpos[sub];
  in.end_hint = subpos[sub + 1];
  return in;
}

__global__ __launch_bounds__(kThreads) void decode_kernel(const DecodeArgs a) {
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_rows = min(a.n_luts - 1, kMaxDecodeRows);
  uint8_t* lds_tables = lds;
  uint8_t* lds_rows = lds + kTablesBytes;
  uint8_t* stage = lds_rows + (kMaxDecodeRows + 1) * 256 + (size_t)wave * a.stage_cap;
  {
    const uint4* src = reinterpret_cast<const uint4*>(a.ws + kWsTablesOffset);
    uint4* dst = reinterpret_cast<uint4*>(lds_tables);
    for (int i = tid; i < kTablesBytes / 16; i += kThreads) dst[i] = src[i];
    stage_rows(a.luts, a.n_luts, n_rows, lds_rows, tid, kThreads);
  }
  __syncthreads();   // the only workgroup barrier: tables are read-only from here on

  const Tables t{lds_tables + kDecOffset, lds_tables + kCntTailOffset};
  const Luts l{lds_rows, n_rows};
  const int64_t n_gap_bytes = a.n_blocks * kGapBytesPerBlock;
  const uint32_t* subpos = reinterpret_cast<const uint32_t*>(a.ws + kWsSubposOffset);
  const bool vec_ok = a.vec_ok != 0;
  const int64_t stride = (int64_t)gridDim.x * kWavesPerGroup;

  int64_t sub = (int64_t)blockIdx.x * kWavesPerGroup + wave;
  if (sub >= a.n_subs) return;
  SubInputs cur = fetch_sub(a, subpos, sub, lane, n_gap_bytes);

  for (; sub < a.n_subs; sub += stride) {
    // ---- requests whose latency the two decode passes hide: the next
    // sub-block's inputs and this one's sign|mantissa bytes
    const int64_t next_sub = sub + stride;
    SubInputs nxt = cur;
    if (next_sub < a.n_subs) nxt = fetch_sub(a, subpos, next_sub, lane, n_gap_bytes);

    const int64_t base = cur.base;
    const int64_t a0 = base & ~(int64_t)(kGroup - 1);
    int64_t end_hint = cur.end_hint;
    if (end_hint > a.n_elements) end_hint = a.n_elements;
    const uint32_t first_body = (base != a0) ? 1u : 0u;   // group 0 is a partial head unless aligned
    U32x2 m[kPrefetchGroups];
#pragma unroll
    for (int k = 0; k < kPrefetchGroups; ++k) {
      m[k] = U32x2{0, 0};
      const int64_t e0 = a0 + (int64_t)(first_body + lane + kLanes * k) * kGroup;
      if (vec_ok && e0 + kGroup <= end_hint) m[k] = load_as<U32x2>(a.sign_mantissa + e0);
    }

    // ---- pass 1 and the exclusive offsets inside the wavefront
    const uint32_t count = count_chunk(t, l, cur.c.hi, cur.c.lo, cur.c.next, cur.gap);
    const uint32_t incl = wave_inclusive_scan(count);
    const uint32_t total = wave_total(incl);
    const uint32_t excl = incl - count;

    // ---- pass 2: decode into this wavefront's staging area, in output order
    const SubPlan p = plan_sub(base, total, a.n_elements, a.stage_cap);
    emit_chunk(t, l, cur.c.hi, cur.c.lo, cur.c.next, cur.gap, thread_quota(excl, count, p.n_out),
               stage + p.phase + excl);
    // Staging is exchanged between the lanes of one wavefront only; its LDS
    // operations execute in order, the fence keeps the compiler from reordering.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- stream out
    const SubSpans sp = spans_of(p);
    if (vec_ok) {
      for (uint32_t i = sp.head_begin + lane; i < sp.head_end; i += kLanes)
        stream_element(i, p, stage, a.sign_mantissa, a.out);
      uint32_t g = sp.body_begin + lane;
#pragma unroll
      for (int k = 0; k < kPrefetchGroups; ++k, g += kLanes) {
        if (g < sp.body_end) {
          // requested early only when the hint covered the group; the hint is the
          // next sub-block's start, which equals this one's end for a valid stream
          const int64_t e0 = p.a0 + (int64_t)g * kGroup;
          const bool early = sp.body_begin == first_body && e0 + kGroup <= end_hint;
          const U32x2 mm = early ? m[k] : load_as<U32x2>(a.sign_mantissa + e0);
          stream_group(g, p, stage, mm, a.out);
        }
      }
      for (; g < sp.body_end; g += kLanes)
        stream_group(g, p, stage, load_as<U32x2>(a.sign_mantissa + p.a0 + (int64_t)g * kGroup), a.out);
      for (uint32_t i = sp.tail_begin + lane; i < sp.tail_end; i += kLanes)
        stream_element(i, p, stage, a.sign_mantissa, a.out);
    } else {
      for (uint32_t i = p.phase + lane; i < p.phase + p.n_out; i += kLanes)
        stream_element(i, p, stage, a.sign_mantissa, a.out);
    }
    // The next sub-block's staging stores must not pass this one's loads.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    cur = nxt;
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

constexpr int kFixedLds = kTablesBytes + (kMaxDecodeRows + 1) * 256;
constexpr int kLdsPerCu = 160 * 1024;

int groups_per_cu(size_t lds_bytes) {
  int n = (int)(kLdsPerCu / lds_bytes);
  if (n > 4) n = 4;     // 2048 threads per CU
  return n < 1 ? 1 : n;
}

}  // namespace

extern "C" {

int df11_version(void) { return 2; }

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

  hipLaunchKernelGGL(build_tables_kernel, dim3(kTableEntries / 256), dim3(256), 0, s, luts, (int)n_luts,
                     ws, (uint32_t)n_blocks);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);

  if (n_blocks > 0) {
    IndexArgs a;
    a.luts = luts;
    a.codes = encoded_exponent;
    a.positions = output_positions;
    a.gaps = gaps;
    a.ws = ws;
    a.n_bytes = n_bytes;
    a.n_elements = n_elements;
    a.n_blocks = n_blocks;
    a.n_luts = n_luts;
    a.codes_aligned = (reinterpret_cast<uintptr_t>(encoded_exponent) & 7) == 0;
    const size_t lds_bytes = (size_t)kFixedLds + 64;
    int64_t grid = (int64_t)info.cus * groups_per_cu(lds_bytes);
    if (grid > n_blocks) grid = n_blocks;
    hipLaunchKernelGGL(index_kernel, dim3((unsigned)grid), dim3(kThreads), lds_bytes, s, a);
    e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e);
  }
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
                int32_t n_luts, int64_t n_bytes, int64_t n_elements, const void* workspace,
                int32_t max_elems_per_subblock, void* stream) {
  (void)output_positions;   // superseded by the sub-block positions in the workspace
  if (n_bytes < 0 || n_elements < 0 || n_luts < 2) return DF11_ERR_INVALID_ARGUMENT;
  if (n_bytes == 0 || n_elements == 0) return DF11_OK;
  if (!luts || !encoded_exponent || !sign_mantissa || !gaps || !outputs || !workspace)
    return DF11_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(workspace) & 15) || (reinterpret_cast<uintptr_t>(outputs) & 1))
    return DF11_ERR_INVALID_ARGUMENT;
  if (max_elems_per_subblock <= 0 || max_elems_per_subblock > kMaxElemsPerSub)
    max_elems_per_subblock = kMaxElemsPerSub;

  DeviceInfo info;
  if (int rc = device_info(info)) return rc;

  DecodeArgs a;
  a.luts = luts;
  a.codes = encoded_exponent;
  a.sign_mantissa = sign_mantissa;
  a.gaps = gaps;
  a.out = outputs;
  a.ws = static_cast<const uint8_t*>(workspace);
  a.n_bytes = n_bytes;
  a.n_elements = n_elements;
  a.n_blocks = (n_bytes + kBlockBytes - 1) / kBlockBytes;
  a.n_subs = (n_bytes + kSubBytes - 1) / kSubBytes;
  a.n_luts = n_luts;
  a.stage_cap = ((max_elems_per_subblock + kGroup + 15) / 16) * 16;   // + up to 7 elements of output phase
  a.codes_aligned = (reinterpret_cast<uintptr_t>(encoded_exponent) & 7) == 0;
  a.vec_ok = (reinterpret_cast<uintptr_t>(sign_mantissa) & 7) == 0 &&
             (reinterpret_cast<uintptr_t>(outputs) & 15) == 0;

  const size_t lds_bytes = (size_t)kFixedLds + (size_t)kWavesPerGroup * (size_t)a.stage_cap;
  int64_t grid = (int64_t)info.cus * groups_per_cu(lds_bytes);
  const int64_t needed = (a.n_subs + kWavesPerGroup - 1) / kWavesPerGroup;
  if (grid > needed) grid = needed;

  hipLaunchKernelGGL(decode_kernel, dim3((unsigned)grid), dim3(kThreads), lds_bytes,
                     static_cast<hipStream_t>(stream), a);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DF11_OK : hip_fail(e);
}

}  // extern "C"
