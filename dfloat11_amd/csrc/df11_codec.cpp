// Host-side DF11 codec: exponent histogram, prefix-code construction, byte-LUT
// layout and the multi-threaded bit packer.  Plain C++17, no GPU dependency.
//
// The code construction differs from the reference's (a heap Huffman from a
// third-party package followed by a flattening heuristic): lengths come from a
// Huffman pass and, when the 32-bit limit or the LUT layout's limits are hit,
// from package-merge (optimal length-limited codes); code words are assigned
// canonically.  The stream stays decodable by any DF11 decoder because the file
// carries its own LUTs.
#include <algorithm>
#include <array>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <queue>
#include <thread>
#include <vector>

#include "../../include/df11.h"

namespace {

constexpr int kSymbols = 256;
constexpr int kEof = 256;          // leaf id of the end-of-stream pseudo-symbol
constexpr int kEsc = 257;          // leaf id of the escape that carries symbols >= 240
constexpr int kPointerFloor = 240; // LUT values >= 240 are read as pointers on levels 0..2
constexpr int kMaxSubLuts = 16;
constexpr int64_t kChunkBits = 64;
constexpr int64_t kBlockBits = 8 * DF11_BLOCK_BYTES;

struct Leaf {
  int id;
  uint64_t weight;
  int len = 0;
};

// ---- parallel helper ---------------------------------------------------------
int pick_threads(int32_t requested, int64_t n, int64_t min_per_thread) {
  int hw = (int)std::thread::hardware_concurrency();
  if (hw <= 0) hw = 1;
  // hardware_concurrency() reports the machine, not the share this process may
  // use; honour the usual environment knobs and stay modest by default.
  for (const char* name : {"DF11_NUM_THREADS", "OMP_NUM_THREADS"}) {
    if (const char* v = std::getenv(name)) {
      const int k = std::atoi(v);
      if (k > 0) {
        hw = k;
        break;
      }
    }
  }
  if (hw > 64) hw = 64;
  int t = requested > 0 ? requested : hw;
  int64_t cap = n / min_per_thread;
  if (cap < 1) cap = 1;
  if (t > cap) t = (int)cap;
  return t;
}

template <class F>
void parallel_for(int n_threads, F&& body) {   // body(thread_index)
  if (n_threads <= 1) {
    body(0);
    return;
  }
  std::vector<std::thread> pool;
  pool.reserve(n_threads);
  for (int t = 0; t < n_threads; ++t) pool.emplace_back([&body, t] { body(t); });
  for (auto& th : pool) th.join();
}

// ---- code lengths --------------------------------------------------------------
// Plain Huffman lengths; ties broken by leaf id so the result is deterministic.
void huffman_lengths(std::vector<Leaf>& leaves) {
  const int n = (int)leaves.size();
  if (n == 1) {
    leaves[0].len = 1;
    return;
  }
  struct Node {
    uint64_t w;
    int order;
    int idx;
  };
  auto cmp = [](const Node& a, const Node& b) { return a.w != b.w ? a.w > b.w : a.order > b.order; };
  std::priority_queue<Node, std::vector<Node>, decltype(cmp)> heap(cmp);
  std::vector<int> parent(2 * n, -1);
  for (int i = 0; i < n; ++i) heap.push({leaves[i].weight, i, i});
  int next = n;
  while (heap.size() > 1) {
    Node a = heap.top();
    heap.pop();
    Node b = heap.top();
    heap.pop();
    parent[a.idx] = next;
    parent[b.idx] = next;
    heap.push({a.w + b.w, next, next});
    ++next;
  }
  for (int i = 0; i < n; ++i) {
    int d = 0;
    for (int p = parent[i]; p != -1; p = parent[p]) ++d;
    leaves[i].len = d;
  }
}

// Package-merge: optimal lengths under len <= max_len.  Requires 2^max_len >= n.
void package_merge_lengths(std::vector<Leaf>& leaves, int max_len) {
  const int n = (int)leaves.size();
  if (n == 1) {
    leaves[0].len = 1;
    return;
  }
  std::vector<int> order(n);
  for (int i = 0; i < n; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(),
                   [&](int a, int b) { return leaves[a].weight < leaves[b].weight; });
  struct Item {
    uint64_t w;
    std::vector<uint16_t> uses;   // how many times each leaf occurs in the package
  };
  auto leaf_items = [&] {
    std::vector<Item> v(n);
    for (int k = 0; k < n; ++k) {
      v[k].w = leaves[order[k]].weight;
      v[k].uses.assign(n, 0);
      v[k].uses[order[k]] = 1;
    }
    return v;
  };
  std::vector<Item> prev = leaf_items();
  for (int level = 1; level < max_len; ++level) {
    std::vector<Item> packaged;
    for (size_t i = 0; i + 1 < prev.size(); i += 2) {
      Item p;
      p.w = prev[i].w + prev[i + 1].w;
      p.uses = prev[i].uses;
      for (int k = 0; k < n; ++k) p.uses[k] += prev[i + 1].uses[k];
      packaged.push_back(std::move(p));
    }
    std::vector<Item> base = leaf_items(), merged;
    merged.reserve(base.size() + packaged.size());
    size_t i = 0, j = 0;
    while (i < base.size() || j < packaged.size()) {
      if (j >= packaged.size() || (i < base.size() && base[i].w <= packaged[j].w))
        merged.push_back(std::move(base[i++]));
      else
        merged.push_back(std::move(packaged[j++]));
    }
    prev = std::move(merged);
  }
  for (auto& l : leaves) l.len = 0;
  for (int k = 0; k < 2 * n - 2; ++k)
    for (int s = 0; s < n; ++s) leaves[s].len += prev[k].uses[s];
}

// Canonical code words: leaves ordered by (length, id), consecutive values.
void assign_canonical(std::vector<Leaf>& leaves, std::vector<uint32_t>& codes) {
  const int n = (int)leaves.size();
  std::vector<int> order(n);
  for (int i = 0; i < n; ++i) order[i] = i;
  std::sort(order.begin(), order.end(), [&](int a, int b) {
    return leaves[a].len != leaves[b].len ? leaves[a].len < leaves[b].len : leaves[a].id < leaves[b].id;
  });
  codes.assign(n, 0);
  uint64_t code = 0;
  int prev_len = leaves[order[0]].len;
  for (int k = 0; k < n; ++k) {
    const int i = order[k];
    code <<= (leaves[i].len - prev_len);
    prev_len = leaves[i].len;
    codes[i] = (uint32_t)code;
    ++code;
  }
}

// ---- LUT layout ------------------------------------------------------------------
struct Prefix {
  int level;
  uint32_t value;
  bool operator==(const Prefix& o) const { return level == o.level && value == o.value; }
  bool operator<(const Prefix& o) const { return level != o.level ? level < o.level : value < o.value; }
};

// Sub-tables a code set needs: every (level, first 8*level bits) of every code
// longer than 8*level bits, levels 1..3.  Rows are ordered by level, then by
// prefix value (the order a stable sort by prefix length gives to a table listed
// in code-word order).
std::vector<Prefix> collect_prefixes(const uint8_t* code_len, const uint32_t* code_val) {
  std::vector<Prefix> p;
  p.push_back({0, 0});
  for (int s = 0; s < kSymbols; ++s) {
    const int l = code_len[s];
    if (!l) continue;
    for (int level = 1; level <= (l - 1) / 8; ++level) p.push_back({level, code_val[s] >> (l - 8 * level)});
  }
  std::sort(p.begin(), p.end());
  p.erase(std::unique(p.begin(), p.end()), p.end());
  return p;
}

int check_layout(const uint8_t* code_len, const uint32_t* code_val) {
  for (int s = 0; s < kSymbols; ++s) {
    const int l = code_len[s];
    if (l > 32) return DF11_ERR_FORMAT;
    if (l && s >= kPointerFloor && l <= 24) return DF11_ERR_FORMAT;
  }
  if ((int)collect_prefixes(code_len, code_val).size() - 1 > kMaxSubLuts) return DF11_ERR_FORMAT;
  return DF11_OK;
}

struct Code {
  uint8_t len[kSymbols] = {};
  uint32_t val[kSymbols] = {};
  int eof_len = 0;
  uint32_t eof_val = 0;
};

// One attempt at a code with main-code lengths capped at max_len (0 = plain Huffman).
bool try_build(const uint64_t* hist, int max_len, Code& out) {
  std::vector<Leaf> main_leaves, members;
  uint64_t esc_weight = 1;   // the end-of-stream leaf
  bool has_high = false;
  for (int s = 0; s < kSymbols; ++s) {
    if (!hist[s]) continue;
    if (s >= kPointerFloor) {
      has_high = true;
      esc_weight += hist[s];
      members.push_back({s, hist[s]});
    } else {
      main_leaves.push_back({s, hist[s]});
    }
  }
  if (has_high) {
    members.push_back({kEof, 1});
    main_leaves.push_back({kEsc, esc_weight});
    if (max_len == 0 || max_len > 24) max_len = 24;   // the escape must end by bit 24
  } else {
    main_leaves.push_back({kEof, 1});
  }
  int need = 1;
  while ((1 << need) < (int)main_leaves.size()) ++need;
  if (max_len && max_len < need) return false;
  if (max_len == 0) {
    huffman_lengths(main_leaves);
    for (auto& l : main_leaves)
      if (l.len > 32) return false;
  } else {
    package_merge_lengths(main_leaves, max_len);
  }
  std::vector<uint32_t> main_codes;
  assign_canonical(main_leaves, main_codes);

  out = Code();
  int esc_len = 0;
  uint32_t esc_val = 0;
  for (size_t i = 0; i < main_leaves.size(); ++i) {
    const Leaf& l = main_leaves[i];
    if (l.id == kEof) {
      out.eof_len = l.len;
      out.eof_val = main_codes[i];
    } else if (l.id == kEsc) {
      esc_len = l.len;
      esc_val = main_codes[i];
    } else {
      out.len[l.id] = (uint8_t)l.len;
      out.val[l.id] = main_codes[i];
    }
  }
  if (has_high) {
    // Members sit below bit 24 of the escape path: escape code, zero bits up to
    // bit 24, then a 1..8-bit sub-code.  Every member is therefore 25..32 bits
    // long and resolves on the fourth LUT level, which no decoder re-tests.
    if (members.size() == 1) {
      members[0].len = 1;
    } else {
      huffman_lengths(members);
      bool too_long = false;
      for (auto& m : members) too_long |= m.len > 8;
      if (too_long) package_merge_lengths(members, 8);
    }
    std::vector<uint32_t> sub_codes;
    assign_canonical(members, sub_codes);
    const uint32_t stem = esc_val << (24 - esc_len);
    for (size_t i = 0; i < members.size(); ++i) {
      const int len = 24 + members[i].len;
      const uint32_t val = (stem << members[i].len) | sub_codes[i];
      if (members[i].id == kEof) {
        out.eof_len = len;
        out.eof_val = val;
      } else {
        out.len[members[i].id] = (uint8_t)len;
        out.val[members[i].id] = val;
      }
    }
  }
  return check_layout(out.len, out.val) == DF11_OK;
}

}  // namespace

extern "C" {

int df11_histogram(const uint16_t* w, int64_t n, uint64_t hist[256], int32_t n_threads) {
  if ((!w && n > 0) || n < 0 || !hist) return DF11_ERR_INVALID_ARGUMENT;
  const int T = pick_threads(n_threads, n, 1 << 16);
  std::vector<std::array<uint64_t, 256>> part(T);
  parallel_for(T, [&](int t) {
    part[t].fill(0);
    const int64_t lo = n * t / T, hi = n * (t + 1) / T;
    for (int64_t i = lo; i < hi; ++i) part[t][(w[i] >> 7) & 0xff]++;
  });
  for (int s = 0; s < 256; ++s) {
    hist[s] = 0;
    for (int t = 0; t < T; ++t) hist[s] += part[t][s];
  }
  return DF11_OK;
}

int df11_split(const uint16_t* w, int64_t n, uint8_t* exponent, uint8_t* sign_mantissa,
               int32_t n_threads) {
  if (n < 0 || (n > 0 && (!w || !exponent || !sign_mantissa))) return DF11_ERR_INVALID_ARGUMENT;
  const int T = pick_threads(n_threads, n, 1 << 16);
  parallel_for(T, [&](int t) {
    const int64_t lo = n * t / T, hi = n * (t + 1) / T;
    for (int64_t i = lo; i < hi; ++i) {
      const uint32_t v = w[i];
      exponent[i] = (uint8_t)(v >> 7);
      sign_mantissa[i] = (uint8_t)(((v >> 8) & 0x80u) | (v & 0x7fu));
    }
  });
  return DF11_OK;
}

int df11_build_code(const uint64_t hist[256], uint8_t code_len[256], uint32_t code_val[256],
                    int32_t* eof_len, uint32_t* eof_val) {
  if (!hist || !code_len || !code_val || !eof_len || !eof_val) return DF11_ERR_INVALID_ARGUMENT;
  bool any = false;
  for (int s = 0; s < 256; ++s) any |= hist[s] != 0;
  if (!any) return DF11_ERR_INVALID_ARGUMENT;
  // Plain Huffman first; then optimal length-limited codes with a shrinking
  // cap until the layout limits hold.  A cap of 8 always does: at most 240
  // symbols plus one extra leaf fit in 8 bits and need three sub-tables at most.
  static const int caps[] = {0, 32, 28, 24, 20, 16, 14, 12, 11, 10, 9, 8};
  Code c;
  for (int cap : caps) {
    if (try_build(hist, cap, c)) {
      std::memcpy(code_len, c.len, sizeof c.len);
      std::memcpy(code_val, c.val, sizeof c.val);
      *eof_len = c.eof_len;
      *eof_val = c.eof_val;
      return DF11_OK;
    }
  }
  return DF11_ERR_FORMAT;
}

int df11_build_luts(const uint8_t code_len[256], const uint32_t code_val[256], uint8_t* luts,
                    int32_t cap_rows, int32_t* n_luts) {
  if (!code_len || !code_val || !luts || !n_luts) return DF11_ERR_INVALID_ARGUMENT;
  if (int rc = check_layout(code_len, code_val)) return rc;
  const std::vector<Prefix> prefixes = collect_prefixes(code_len, code_val);
  const int n_rows = (int)prefixes.size();
  if (n_rows + 1 > cap_rows) return DF11_ERR_CAPACITY;

  // Unset entries (the end-of-stream code's slots, unused code space) inherit
  // the most recent symbol entry, carried from row to row; before the first one
  // that is the symbol below 240 with the shortest code.  On the first three
  // levels a decoder reads values of 240 and above as pointers, so only symbols
  // below 240 may fill there; a code without any (every exponent >= 240) fills
  // those rows with the row's own first pointer instead.  Any bit pattern,
  // padding included, therefore decodes to a symbol of non-zero length without
  // leaving the rows that exist.
  int carried = -1;
  for (int s = 0; s < kPointerFloor; ++s)
    if (code_len[s] && (carried < 0 || code_len[s] < code_len[carried])) carried = s;
  bool any = false;
  for (int s = 0; s < kSymbols; ++s) any |= code_len[s] != 0;
  if (!any) return DF11_ERR_INVALID_ARGUMENT;

  for (int pi = 0; pi < n_rows; ++pi) {
    const Prefix& p = prefixes[pi];
    int entry[256];
    bool is_pointer[256] = {};
    std::fill(entry, entry + 256, -1);
    for (int s = 0; s < kSymbols; ++s) {
      const int l = code_len[s];
      if (!l || l <= 8 * p.level || (uint32_t)((uint64_t)code_val[s] >> (l - 8 * p.level)) != p.value) continue;   // 64-bit: the shift is 32 for a 32-bit code on level 0
      int key, value;
      if ((l - 1) / 8 == p.level) {
        const int rem = l - 8 * p.level;
        key = (int)((code_val[s] & ((1u << rem) - 1u)) << (8 - rem));
        value = s;
      } else {
        key = (int)((code_val[s] >> (l - 8 * p.level - 8)) & 0xffu);
        const Prefix child{p.level + 1, code_val[s] >> (l - 8 * (p.level + 1))};
        const int row = (int)(std::lower_bound(prefixes.begin(), prefixes.end(), child) - prefixes.begin());
        value = 256 - row;
        is_pointer[key] = true;
      }
      if (entry[key] >= 0 && entry[key] != value) return DF11_ERR_FORMAT;   // not prefix-free
      entry[key] = value;
    }
    int first_own = -1;
    for (int i = 0; i < 256 && first_own < 0; ++i) first_own = entry[i];
    if (first_own < 0) return DF11_ERR_FORMAT;   // a row that no code reaches
    for (int i = 0; i < 256; ++i) {
      if (entry[i] >= 0 && !is_pointer[i]) carried = entry[i];
      const bool usable = carried >= 0 && (p.level == 3 || carried < kPointerFloor);
      luts[pi * 256 + i] = (uint8_t)(entry[i] >= 0 ? entry[i] : usable ? carried : first_own);
    }
  }
  std::memcpy(luts + n_rows * 256, code_len, 256);
  *n_luts = n_rows + 1;
  return DF11_OK;
}

int df11_encode_size(const uint8_t* exponent, int64_t n, const uint8_t code_len[256],
                     int64_t* n_bytes, int64_t* n_blocks, int32_t n_threads) {
  if (n < 0 || (n > 0 && !exponent) || !code_len || !n_bytes || !n_blocks) return DF11_ERR_INVALID_ARGUMENT;
  const int T = pick_threads(n_threads, n, 1 << 16);
  std::vector<int64_t> bits(T, 0);
  std::vector<int> bad(T, 0);
  parallel_for(T, [&](int t) {
    const int64_t lo = n * t / T, hi = n * (t + 1) / T;
    int64_t b = 0;
    for (int64_t i = lo; i < hi; ++i) {
      const int l = code_len[exponent[i]];
      bad[t] |= (l == 0);
      b += l;
    }
    bits[t] = b;
  });
  int64_t total = 0;
  for (int t = 0; t < T; ++t) {
    if (bad[t]) return DF11_ERR_INVALID_ARGUMENT;   // a symbol without a code
    total += bits[t];
  }
  *n_bytes = (total + 7) / 8;
  *n_blocks = (*n_bytes + DF11_BLOCK_BYTES - 1) / DF11_BLOCK_BYTES;
  return DF11_OK;
}

int df11_encode(const uint8_t* exponent, int64_t n, const uint8_t code_len[256],
                const uint32_t code_val[256], int32_t eof_len, uint32_t eof_val, uint8_t* encoded,
                int64_t n_bytes, uint8_t* gaps, uint32_t* output_positions, int64_t n_blocks,
                int32_t n_threads) {
  if (n < 0 || n_bytes < 0 || n_blocks < 0 || !code_len || !code_val || !output_positions)
    return DF11_ERR_INVALID_ARGUMENT;
  if (n > 0 && (!exponent || !encoded || !gaps)) return DF11_ERR_INVALID_ARGUMENT;
  if (n >= ((int64_t)1 << 32)) return DF11_ERR_UNSUPPORTED;   // output_positions is u32
  if (eof_len < 0 || eof_len > 32) return DF11_ERR_INVALID_ARGUMENT;

  const int T = pick_threads(n_threads, n, 1 << 16);
  // bit offset at which each thread's slice starts
  std::vector<int64_t> start_bit(T + 1, 0);
  {
    std::vector<int64_t> bits(T, 0);
    parallel_for(T, [&](int t) {
      const int64_t lo = n * t / T, hi = n * (t + 1) / T;
      int64_t b = 0;
      for (int64_t i = lo; i < hi; ++i) b += code_len[exponent[i]];
      bits[t] = b;
    });
    for (int t = 0; t < T; ++t) start_bit[t + 1] = start_bit[t] + bits[t];
  }
  const int64_t total_bits = start_bit[T];
  if ((total_bits + 7) / 8 != n_bytes) return DF11_ERR_CAPACITY;
  if ((n_bytes + DF11_BLOCK_BYTES - 1) / DF11_BLOCK_BYTES != n_blocks) return DF11_ERR_CAPACITY;

  const int64_t n_chunks = n_blocks * DF11_THREADS_PER_BLOCK;
  std::vector<uint8_t> gap_vals((size_t)n_chunks, 0);
  std::memset(encoded, 0, (size_t)n_bytes);
  // every block without a code start (only a trailing one can lack it) and the
  // sentinel point at the end of the data
  for (int64_t b = 0; b <= n_blocks; ++b) output_positions[b] = (uint32_t)n;

  parallel_for(T, [&](int t) {
    const int64_t lo = n * t / T, hi = n * (t + 1) / T;
    if (lo >= hi) return;
    int64_t pos = start_bit[t];
    // start of the previous code, to tell whether this slice's first code is the
    // first one in its chunk / block
    int64_t prev_start = lo > 0 ? pos - code_len[exponent[lo - 1]] : -1;
    int64_t byte = pos >> 3;
    const int64_t first_byte = byte, last_byte = (start_bit[t + 1] - 1) >> 3;
    uint64_t acc = 0;         // pending bits, right-aligned
    int n_acc = (int)(pos & 7);
    auto put = [&](uint8_t v) {
      if (byte == first_byte || byte == last_byte)
        __atomic_fetch_or(&encoded[byte], v, __ATOMIC_RELAXED);   // shared with a neighbouring slice
      else
        encoded[byte] = v;
      ++byte;
    };
    for (int64_t i = lo; i < hi; ++i) {
      const uint8_t s = exponent[i];
      const int l = code_len[s];
      if (prev_start < 0 || (pos / kChunkBits) != (prev_start / kChunkBits)) {
        gap_vals[(size_t)(pos / kChunkBits)] = (uint8_t)(pos % kChunkBits);
        if (prev_start < 0 || (pos / kBlockBits) != (prev_start / kBlockBits))
          output_positions[pos / kBlockBits] = (uint32_t)i;
      }
      prev_start = pos;
      acc = (acc << l) | code_val[s];
      n_acc += l;
      pos += l;
      while (n_acc >= 8) {
        put((uint8_t)(acc >> (n_acc - 8)));
        n_acc -= 8;
      }
      acc &= (1ull << n_acc) - 1ull;
    }
    if (n_acc > 0) put((uint8_t)(acc << (8 - n_acc)));
  });

  // Tail: the last partial byte is completed with the leading bits of the
  // end-of-stream code, which also counts as a code start for gaps/positions.
  if (total_bits % 8 != 0) {
    const int64_t pos = total_bits;
    const int64_t prev_start = pos - code_len[exponent[n - 1]];
    if (pos / kChunkBits != prev_start / kChunkBits) {
      gap_vals[(size_t)(pos / kChunkBits)] = (uint8_t)(pos % kChunkBits);
      if (pos / kBlockBits != prev_start / kBlockBits) output_positions[pos / kBlockBits] = (uint32_t)n;
    }
    const int room = 8 - (int)(pos & 7);
    const uint32_t fill = eof_len >= room ? (eof_val >> (eof_len - room))
                                          : (eof_len ? (eof_val << (room - eof_len)) : 0u);
    encoded[n_bytes - 1] |= (uint8_t)(fill & ((1u << room) - 1u));
  }

  // 5-bit gaps, MSB-first: eight gaps -> five bytes.
  const int64_t n_groups = n_chunks / 8;
  const int TG = pick_threads(n_threads, n_groups, 1 << 12);
  parallel_for(TG, [&](int t) {
    const int64_t lo = n_groups * t / TG, hi = n_groups * (t + 1) / TG;
    for (int64_t g = lo; g < hi; ++g) {
      uint64_t v = 0;
      for (int k = 0; k < 8; ++k) v = (v << 5) | (gap_vals[(size_t)(g * 8 + k)] & 31u);
      for (int k = 0; k < 5; ++k) gaps[g * 5 + k] = (uint8_t)(v >> (32 - 8 * k));
    }
  });
  return DF11_OK;
}

}  // extern "C"
