// Mutation fuzz of the burnpack container parser (burn_amd/csrc/pack_format.hpp), CPU only.
//
//   g++ -std=c++17 -O1 -g -fsanitize=address,undefined -fno-sanitize-recover=all
//       -I include -I burn_amd/csrc tests/cpp/fuzz_pack.cpp -o fuzz_pack
//   fuzz_pack [cases] [seed] [reference-written .bpk ...]
//
// Seeds: containers this file assembles with the library's own CBOR writer (float and quantized
// entries, user metadata), plus any files named on the command line. Every case is one seed with a
// few mutations (bit flips, byte overwrites, truncations, length fields blown up, spliced runs) fed
// to parse_container. The parser must answer each with a status -- never a crash, a sanitizer
// report or an exception -- and whatever it accepts must describe bytes the container really holds
// (the limits of crates/burn-pack/src/reader.rs; reject cases as crates/burn-pack/tests/errors.rs).
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iterator>
#include <memory>

#include "pack_format.hpp"

using namespace bq::pack;

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint64_t rnd() {  // splitmix64
  uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

struct Desc {
  std::string name;
  const char* dtype;    // nullptr: QFloat with `scheme`
  bq_scheme scheme;
  std::vector<uint64_t> shape;
  size_t bytes;
  bool param;
};

static std::vector<uint8_t> assemble(const std::vector<Desc>& tensors, bool with_metadata) {
  std::vector<uint64_t> begin(tensors.size()), end(tensors.size());
  uint64_t cur = 0;
  for (size_t i = 0; i < tensors.size(); ++i) {
    begin[i] = align_up(cur, kAlign);
    end[i] = begin[i] + tensors[i].bytes;
    cur = end[i];
  }
  CborWriter c;
  c.map(with_metadata ? 2 : 1);
  c.text("tensors");
  c.map(tensors.size());
  for (size_t i = 0; i < tensors.size(); ++i) {
    const Desc& t = tensors[i];
    c.text(t.name);
    c.map(t.param ? 4 : 3);
    c.text("dtype");
    if (t.dtype) { c.text(t.dtype); } else { c.map(1); c.text("QFloat"); write_scheme(c, t.scheme); }
    c.text("shape");
    c.array(t.shape.size());
    for (uint64_t d : t.shape) c.uint(d);
    c.text("data_offsets");
    c.array(2);
    c.uint(begin[i]);
    c.uint(end[i]);
    if (t.param) { c.text("param_id"); c.uint(0x1234567890ABCDEFull + i); }
  }
  if (with_metadata) {
    c.text("metadata");
    c.map(2);
    c.text("format"); c.text("burnpack");
    c.text("producer"); c.text("fuzz");
  }
  const size_t msize = c.out.size();
  const size_t start = static_cast<size_t>(align_up(kHeader + msize, kAlign));
  std::vector<uint8_t> out(start + static_cast<size_t>(cur), 0);
  const uint8_t header[kHeader] = {0x4E, 0x52, 0x55, 0x42, 0x01, 0x00, static_cast<uint8_t>(msize), static_cast<uint8_t>(msize >> 8),
                                   static_cast<uint8_t>(msize >> 16), static_cast<uint8_t>(msize >> 24)};
  memcpy(out.data(), header, kHeader);
  memcpy(out.data() + kHeader, c.out.data(), msize);
  for (size_t i = static_cast<size_t>(start); i < out.size(); ++i) out[i] = static_cast<uint8_t>(i * 131);
  return out;
}

// What an accepted container must satisfy, whatever was done to its bytes.
static bool check_accepted(const Index& ix, size_t size, const char** why) {
  if (ix.entries.size() > kMaxTensors) { *why = "more tensors than the limit"; return false; }
  for (size_t i = 0; i < ix.entries.size(); ++i) {
    const Entry& e = ix.entries[i];
    if (e.end < e.begin) { *why = "inverted offsets"; return false; }
    if (e.end - e.begin > kMaxTensorBytes) { *why = "tensor over the size limit"; return false; }
    if (e.end > e.begin && (ix.data_start > size || e.end > size - ix.data_start)) { *why = "tensor bytes outside the container"; return false; }
    if (e.dtype < 0 || e.dtype > BQ_PACK_QFLOAT) { *why = "dtype out of range"; return false; }
    if (i > 0 && ix.entries[i - 1].name > e.name) { *why = "entries not in name order"; return false; }
    // touch every byte the descriptor claims (the sanitizer sees an out-of-range read)
  }
  return true;
}

int main(int argc, char** argv) {
  const long cases = argc > 1 ? atol(argv[1]) : 100000;
  if (argc > 2) rng_state ^= strtoull(argv[2], nullptr, 0);
  std::vector<std::vector<uint8_t>> seeds;
  {
    bq_scheme q8{};   // Q8S, block [32], packed, f32 scales
    q8.value = BQ_Q8S; q8.level = BQ_LEVEL_BLOCK; q8.store = BQ_STORE_PACKED_U32; q8.block_rank = 1; q8.block[0] = 32;
    bq_scheme q4{};   // Q4S per tensor, two-level flag set, f16 scales
    q4.value = BQ_Q4S; q4.level = BQ_LEVEL_BLOCK; q4.store = BQ_STORE_NATIVE; q4.scale_dtype = BQ_SCALE_F16; q4.block_rank = 2;
    q4.block[0] = 2; q4.block[1] = 16; q4.tensor_scale = 1;
    seeds.push_back(assemble({{"w", "F32", {}, {2, 3}, 24, false}}, false));
    seeds.push_back(assemble({{"a.weight", "F32", {}, {4, 8}, 128, true}, {"a.bias", "BF16", {}, {8}, 16, true},
                              {"q.weight", nullptr, q8, {64, 64}, 64 * 64 + 4 * 128, true}, {"q2", nullptr, q4, {4, 32}, 4 * 32 + 2 * 4 + 4, false},
                              {"empty", "U8", {}, {0}, 0, false}, {"i", "I64", {}, {3}, 24, false}}, true));
    seeds.push_back(assemble({}, true));
  }
  for (int i = 3; i < argc; ++i) {
    std::ifstream f(argv[i], std::ios::binary);
    std::vector<uint8_t> b((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (b.empty()) { fprintf(stderr, "cannot read seed %s\n", argv[i]); return 2; }
    seeds.push_back(std::move(b));
  }
  // the seeds themselves must parse
  for (size_t s = 0; s < seeds.size(); ++s) {
    Index ix; Failure f; const char* why = "";
    if (parse_container(seeds[s].data(), seeds[s].size(), &ix, &f) != BQ_OK || !check_accepted(ix, seeds[s].size(), &why)) {
      fprintf(stderr, "seed %zu rejected: %s %s\n", s, f.message, why);
      return 1;
    }
  }
  long accepted = 0, rejected = 0;
  long by_status[16] = {0};
  for (long c = 0; c < cases; ++c) {
    // (the built seeds are a few hundred bytes; a file seed may be a megabyte, so it takes one case in 16)
    const size_t built = 3;
    std::vector<uint8_t> b = seeds[(seeds.size() > built && rnd() % 16 == 0) ? built + rnd() % (seeds.size() - built) : rnd() % built];
    // mutations concentrate on header + metadata, which is what the parser reads
    const size_t msize = b.size() >= kHeader ? (b[6] | (b[7] << 8) | (static_cast<size_t>(b[8]) << 16)) : 0;
    const size_t hot = std::min(b.size(), kHeader + msize);
    const int n_mut = 1 + static_cast<int>(rnd() % 4);
    for (int m = 0; m < n_mut && !b.empty(); ++m) {
      const size_t at = rnd() % (rnd() % 8 ? std::max<size_t>(std::min(hot, b.size()), 1) : b.size());
      switch (rnd() % 8) {
        case 0: b[at] ^= static_cast<uint8_t>(1u << (rnd() % 8)); break;                 // bit flip
        case 1: b[at] = static_cast<uint8_t>(rnd()); break;                              // random byte
        case 2: b.resize(rnd() % (b.size() + 1)); break;                                 // truncation anywhere
        case 3: b.resize(std::min(b.size(), hot + rnd() % 300)); break;                  // truncation near the data section start
        case 4: {                                                                        // a length / integer head blown up
          static const uint8_t heads[] = {0x1B, 0x3B, 0x5B, 0x7B, 0x9B, 0xBB, 0x9A, 0xBA, 0x7A, 0x99, 0xB9, 0xDB, 0xFB, 0x9F, 0xBF, 0xFF};
          b[at] = heads[rnd() % sizeof(heads)];
          for (size_t i = 1; i <= 8 && at + i < b.size(); ++i)
            if (rnd() % 2) b[at + i] = rnd() % 3 ? 0xFF : static_cast<uint8_t>(rnd());
          break;
        }
        case 5: {                                                                        // a run copied over another place
          const size_t from = rnd() % b.size(), n = std::min<size_t>(rnd() % 64, std::min(b.size() - from, b.size() - at));
          memmove(b.data() + at, b.data() + from, n);
          break;
        }
        case 6: {                                                                        // the header's metadata size field
          const uint32_t v = rnd() % 4 == 0 ? static_cast<uint32_t>(rnd()) : static_cast<uint32_t>(msize + (rnd() % 64) - 32);
          if (b.size() >= kHeader) { b[6] = v & 0xFF; b[7] = (v >> 8) & 0xFF; b[8] = (v >> 16) & 0xFF; b[9] = (v >> 24) & 0xFF; }
          break;
        }
        default: {                                                                       // a nest of arrays / maps / tags
          static const uint8_t kOpen[] = {0x81, 0xA1, 0xC1, 0x9F};
          const uint8_t open = kOpen[rnd() % 4];
          for (size_t i = at; i < std::min(b.size(), at + 1 + rnd() % 400); ++i) b[i] = open;
        }
      }
    }
    Index ix; Failure f; const char* why = "";
    // (an exact-size heap copy, so that a read one byte past the container is a sanitizer report)
    std::unique_ptr<uint8_t[]> exact(new uint8_t[b.size() ? b.size() : 1]);
    if (!b.empty()) memcpy(exact.get(), b.data(), b.size());
    const bq_status st = parse_container(exact.get(), b.size(), &ix, &f);
    if (st < 0 || st > 15) { fprintf(stderr, "case %ld: status %d out of range\n", c, st); return 1; }
    ++by_status[st];
    if (st == BQ_OK) {
      ++accepted;
      if (!check_accepted(ix, b.size(), &why)) { fprintf(stderr, "case %ld: accepted a container with %s\n", c, why); return 1; }
      uint64_t sum = 0;
      for (const Entry& e : ix.entries)
        for (uint64_t i = e.begin; i < e.end; i += 64) sum += exact[ix.data_start + i];
      if (sum == 0xFFFFFFFFFFFFFFFFull) puts("");
    } else {
      ++rejected;
      if (f.message[0] == 0) { fprintf(stderr, "case %ld: rejected without a message\n", c); return 1; }
    }
  }
  // the reader's own limits, as crates/burn-pack/tests/errors.rs states them
  {
    auto header = [](uint16_t version, uint32_t msize) {
      return std::vector<uint8_t>{0x4E, 0x52, 0x55, 0x42, static_cast<uint8_t>(version), static_cast<uint8_t>(version >> 8),
                                  static_cast<uint8_t>(msize), static_cast<uint8_t>(msize >> 8), static_cast<uint8_t>(msize >> 16), static_cast<uint8_t>(msize >> 24)};
    };
    struct { std::vector<uint8_t> bytes; const char* what; } must_fail[] = {
        {std::vector<uint8_t>(4, 0), "too short"}, {header(2, 0), "future version"},
        {header(1, static_cast<uint32_t>(kMaxMetadata) + 1), "oversized metadata claim"}, {header(1, 4096), "metadata past the end"}};
    for (auto& t : must_fail) {
      Index ix; Failure f;
      if (parse_container(t.bytes.data(), t.bytes.size(), &ix, &f) == BQ_OK) { fprintf(stderr, "accepted: %s\n", t.what); return 1; }
    }
    // a metadata block made of one-byte items only: refused by the node budget, in bounded memory
    std::vector<uint8_t> bomb = header(1, 8u << 20);
    bomb.push_back(0x9A); bomb.push_back(0x00); bomb.push_back(0x7F); bomb.push_back(0xFF); bomb.push_back(0xF0);  // array of 8388592
    bomb.resize(kHeader + (8u << 20), 0x80);                                                                      // ... of empty arrays
    Index ix; Failure f;
    if (parse_container(bomb.data(), bomb.size(), &ix, &f) == BQ_OK) { fprintf(stderr, "accepted the node bomb\n"); return 1; }
  }
  printf("fuzz_pack: %ld cases, %ld accepted, %ld rejected (by status:", cases, accepted, rejected);
  for (int i = 0; i < 9; ++i) printf(" %ld", by_status[i]);
  printf("), %zu seeds\n", seeds.size());
  return 0;
}
