// The host codec (dfloat11_amd/csrc/df11_codec.cpp) under AddressSanitizer and
// UndefinedBehaviorSanitizer (test infrastructure): random alphabets, skews,
// sizes and thread counts, and one Fibonacci histogram that reaches 32-bit
// codes; every stream is compared with the oracle's restatement of the
// reference packer and decoded back with its restatement of the reference kernel.  usage: df11_codec_san [cases]
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/df11.h"

extern "C" int df11o_decode_blocks(const uint8_t* luts, const uint8_t* codes, const uint8_t* sign_mantissa,
                                   const uint32_t* position_offsets, const uint8_t* gaps, uint16_t* outputs,
                                   int n_luts, int64_t n_bytes, int64_t n_elements, int64_t n_positions,
                                   int64_t block_begin, int64_t block_end, int64_t stage_elems);

extern "C" int df11o_encode(const uint8_t* data, int64_t n, const uint8_t* code_len, const uint32_t* code_val,
                            int eof_len, uint32_t eof_val, uint8_t* encoded, int64_t cap_bytes, int64_t* n_bytes_out,
                            uint8_t* gaps_packed, int64_t cap_gap_bytes, int64_t* n_gap_bytes_out,
                            uint32_t* positions, int64_t cap_positions, int64_t* n_positions_out);

static uint64_t state = 88172645463325252ull;
static uint64_t rnd() {
  state ^= state << 13;
  state ^= state >> 7;
  state ^= state << 17;
  return state;
}

static int round_trip(const std::vector<uint16_t>& w, int threads, int* max_len) {
  const int64_t n = (int64_t)w.size();
  uint64_t hist[256];
  uint8_t len[256], luts[18 * 256];
  uint32_t val[256], eof_val;
  int32_t eof_len, n_luts;
  if (df11_histogram(w.data(), n, hist, threads)) return 10;
  if (df11_build_code(hist, len, val, &eof_len, &eof_val)) return 11;
  if (df11_build_luts(len, val, luts, 18, &n_luts)) return 12;
  *max_len = 0;
  for (int s = 0; s < 256; ++s) *max_len = len[s] > *max_len ? len[s] : *max_len;
  std::vector<uint8_t> e(n), sm(n);
  if (df11_split(w.data(), n, e.data(), sm.data(), threads)) return 13;
  int64_t n_bytes, n_blocks;
  if (df11_encode_size(e.data(), n, len, &n_bytes, &n_blocks, threads)) return 14;
  std::vector<uint8_t> enc(n_bytes), gaps(n_blocks * DF11_GAP_BYTES_PER_BLOCK);
  std::vector<uint32_t> pos(n_blocks + 1);
  if (df11_encode(e.data(), n, len, val, eof_len, eof_val, enc.data(), n_bytes, gaps.data(), pos.data(), n_blocks,
                  threads))
    return 15;
  {   // the oracle's restatement of the reference packer writes the same bitstream and gaps
    std::vector<uint8_t> o_enc(n_bytes + 16), o_gaps(gaps.size() + 640);
    std::vector<uint32_t> o_pos(n_blocks + 2);
    int64_t o_nb = 0, o_ng = 0, o_np = 0;
    if (df11o_encode(e.data(), n, len, val, eof_len, eof_val, o_enc.data(), (int64_t)o_enc.size(), &o_nb,
                     o_gaps.data(), (int64_t)o_gaps.size(), &o_ng, o_pos.data(), (int64_t)o_pos.size(), &o_np))
      return 18;
    if (o_nb != n_bytes || memcmp(o_enc.data(), enc.data(), (size_t)n_bytes)) return 19;
    if (o_ng != (int64_t)gaps.size() || memcmp(o_gaps.data(), gaps.data(), gaps.size())) return 20;
    if (o_np < n_blocks || memcmp(o_pos.data(), pos.data(), (size_t)n_blocks * 4)) return 21;
  }
  std::vector<uint16_t> out(n, 0xEEEE);
  if (df11o_decode_blocks(luts, enc.data(), sm.data(), pos.data(), gaps.data(), out.data(), n_luts, n_bytes, n,
                          n_blocks + 1, 0, n_blocks, DF11_MAX_ELEMS_PER_BLOCK + 1024))
    return 16;
  return memcmp(out.data(), w.data(), (size_t)n * 2) ? 17 : 0;
}

static uint16_t word(uint8_t exponent, uint8_t sm) {
  return (uint16_t)(((sm & 0x80) << 8) | (exponent << 7) | (sm & 0x7f));
}

int main(int argc, char** argv) {
  const int cases = argc > 1 ? atoi(argv[1]) : 60;
  int bad = 0, max_len = 0;
  for (int c = 0; c < cases; ++c) {
    const int64_t n = 1 + (int64_t)(rnd() % (c % 10 == 0 ? 1500000 : 70000));
    const int k = 1 + (int)(rnd() % 256), skew = (int)(rnd() % 4);
    std::vector<uint8_t> alphabet(k);
    for (auto& a : alphabet) a = (uint8_t)rnd();
    std::vector<uint16_t> w(n);
    for (auto& x : w) {
      const uint64_t r = rnd();
      int idx = skew == 0 ? (int)(r % k) : (int)((r % k) * ((r >> 20) % k) / k);
      if (skew == 3 && (r >> 40) % 7) idx = 0;
      x = word(alphabet[idx % k], (uint8_t)(r >> 50));
    }
    const int rc = round_trip(w, (int)(rnd() % 9), &max_len);
    if (rc) {
      ++bad;
      printf("case %d n=%lld k=%d skew=%d: failure %d\n", c, (long long)n, k, skew, rc);
    }
  }
  {   // Fibonacci counts: the deepest tree a histogram of this size allows
    std::vector<uint16_t> w;
    uint64_t a = 1, b = 2;
    for (int s = 0; s < 33; ++s) {
      for (uint64_t i = 0; i < a; ++i) w.push_back(word((uint8_t)(3 * s + 1), (uint8_t)rnd()));
      const uint64_t t = a + b;
      a = b;
      b = t;
    }
    for (size_t i = w.size() - 1; i > 0; --i) {
      const size_t j = (size_t)(rnd() % (i + 1));
      const uint16_t t = w[i];
      w[i] = w[j];
      w[j] = t;
    }
    const int rc = round_trip(w, 0, &max_len);
    if (rc || max_len < 32) {
      ++bad;
      printf("fibonacci case n=%zu: failure %d, longest code %d\n", w.size(), rc, max_len);
    }
  }
  printf("codec sanitizer run: %d random cases + 1 Fibonacci case (longest code %d bits), %d failures\n", cases,
         max_len, bad);
  return bad != 0;
}
