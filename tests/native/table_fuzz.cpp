// CPU fuzz of the list-launch tables (optimi_amd/csrc/tables.h), built with
// -fsanitize=address,undefined by tests/test_sanitizers.py.
//
// Feeds build_entries adversarial lists - empty lists, empty tensors at the start, in the middle
// and at the end, one-element tensors, sizes one off the 512-element tile and the chunk, tensors
// beyond 2^31 elements, lists of 100,000 tensors, buffers that are not 16-byte aligned - and
// lists that mix fp32 tensors with 16-bit ones (chunks of 4096 and of 8192 elements side by side,
// no Kahan buffer for the fp32 tensors) - and checks what the kernels rely on:
//   * every rejected argument is rejected with the documented status and nothing is written past
//     the entries;
//   * first_chunk is the running sum of the chunk counts, the chunk map names for every chunk the
//     tensor whose range holds it, and the search of a short list (few_lookup) agrees with it;
//   * the tiles the workgroups derive (tile_base, cut off at numel) cover every element of every
//     tensor exactly once.
// Pointers are made-up addresses and are never dereferenced.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "tables.h"

using namespace optimi_tables;

static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static uint64_t rng() {
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return rng_state;
}

#define CHECK(cond, ...)                                              \
  do {                                                                \
    if (!(cond)) {                                                    \
      std::fprintf(stderr, "table_fuzz: %s:%d: ", __FILE__, __LINE__); \
      std::fprintf(stderr, __VA_ARGS__);                              \
      std::fprintf(stderr, "\n");                                     \
      std::exit(1);                                                   \
    }                                                                 \
  } while (0)

constexpr int kThreads = 64, kUnroll = 1;                          // the library's workgroup shape
constexpr int kSub = kChunkBytes / (kThreads * kUnroll * 16);      // workgroups per chunk
constexpr int64_t kMaxChunks = (int64_t)0x7fffffff / kSub;

static int64_t pick_size(int dtype) {
  const int64_t chunk = chunk_elems(dtype), tile = chunk / kSub;
  static const int64_t small[] = {0, 0, 1, 2, 7, 8, 9};
  switch (rng() % 10) {
    case 0: case 1: return small[rng() % 7];
    case 2: return tile + (int64_t)(rng() % 3) - 1;
    case 3: return chunk + (int64_t)(rng() % 3) - 1;
    case 4: return chunk * (int64_t)(1 + rng() % 5) + (int64_t)(rng() % 3) - 1;
    case 5: return (int64_t)(rng() % 100000);
    case 6: return (int64_t)(rng() % 50000000);
    case 7: return ((int64_t)1 << 31) + (int64_t)(rng() % 1000);   // offsets need 64 bits
    default: return (int64_t)(rng() % 3000);
  }
}

// `mixed`: about a third of the tensors are fp32 whatever `dtype` says, and the last array is one
// that only 16-bit tensors have (its pointers for fp32 tensors are null or garbage).
static void check_list(int n_tensors, int dtype, int n_arrays, uint32_t need, bool force_small, bool mixed = false) {
  const uint32_t low_only = mixed ? bit(n_arrays - 1) : 0u;
  std::vector<int> dtypes((size_t)n_tensors, dtype);
  if (mixed)
    for (int t = 0; t < n_tensors; ++t)
      if (rng() % 3 == 0) dtypes[(size_t)t] = OPTIMI_F32;
  std::vector<int64_t> numel((size_t)n_tensors);
  std::vector<std::vector<const void*>> cols((size_t)n_arrays, std::vector<const void*>((size_t)n_tensors));
  std::vector<const void* const*> lists((size_t)n_arrays);
  std::vector<bool> aligned((size_t)n_tensors, true);
  int64_t want_chunks = 0;
  for (int t = 0; t < n_tensors; ++t) {
    const int dt = dtypes[(size_t)t];
    const int eb = elem_bytes(dt);
    numel[(size_t)t] = force_small ? (int64_t)(rng() % 20000) : pick_size(dt);
    want_chunks += chunks_of(numel[(size_t)t], chunk_elems(dt));
    for (int a = 0; a < n_arrays; ++a) {
      uintptr_t addr = 0x100000000ull + (rng() % (1ull << 40)) * 16;
      const bool absent = dt == OPTIMI_F32 && (low_only & bit(a));
      if (absent) {
        addr = rng() % 2 ? 0 : 0x1001;  // must be ignored: null or not even element-aligned
      } else if (rng() % 8 == 0) {
        addr += (uintptr_t)eb * (1 + rng() % 3);
        if (addr % 16 && (need & bit(a))) aligned[(size_t)t] = false;
      }
      cols[(size_t)a][(size_t)t] = (const void*)addr;
    }
  }
  for (int a = 0; a < n_arrays; ++a) lists[(size_t)a] = (need & bit(a)) ? cols[(size_t)a].data() : nullptr;
  std::vector<TensorEntry> entries((size_t)n_tensors + 1);
  const TensorEntry sentinel = {{(void*)0x5a5a, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr}, -77, -78, 0xdeadbeefu, 0xfeedu};
  entries[(size_t)n_tensors] = sentinel;
  int64_t n_chunks = -1;
  const int rc = build_entries(n_tensors, lists.data(), n_arrays, need, numel.data(), mixed ? dtypes.data() : nullptr, dtype,
                               low_only, kMaxChunks, entries.data(), &n_chunks);
  CHECK(std::memcmp(&entries[(size_t)n_tensors], &sentinel, sizeof(sentinel)) == 0, "wrote past the entries");
  if (want_chunks > kMaxChunks) {
    CHECK(rc == OPTIMI_ERR_SIZE, "a launch of %" PRId64 " chunks was not refused (status %d)", want_chunks, rc);
    return;
  }
  CHECK(rc == OPTIMI_OK, "valid list refused with status %d", rc);
  CHECK(n_chunks == want_chunks, "chunk count %" PRId64 " != %" PRId64, n_chunks, want_chunks);
  int64_t running = 0;
  for (int t = 0; t < n_tensors; ++t) {
    const TensorEntry& e = entries[(size_t)t];
    const bool f32 = dtypes[(size_t)t] == OPTIMI_F32;
    const int64_t chunk = chunk_elems(dtypes[(size_t)t]), tile = chunk / kSub;
    CHECK(e.first_chunk == running && e.numel == numel[(size_t)t], "tensor %d: first_chunk/numel", t);
    CHECK(((e.flags & kEntryVec) != 0) == aligned[(size_t)t], "tensor %d: alignment flag", t);
    CHECK(((e.flags & kEntryF32) != 0) == f32 && entry_chunk_elems(e) == chunk, "tensor %d: dtype flag", t);
    CHECK((e.flags & ~(kEntryVec | kEntryF32)) == 0 && e.pad == 0, "tensor %d: stray flag bits", t);
    for (int a = 0; a < kMaxArrays; ++a) {
      const bool present = a < n_arrays && (need & bit(a)) && !(f32 && (low_only & bit(a)));
      CHECK(e.ptr[a] == (present ? cols[(size_t)a][(size_t)t] : nullptr), "tensor %d array %d pointer", t, a);
    }
    running += chunks_of(e.numel, chunk);
    // the tiles of this tensor: consecutive, disjoint, ending exactly at numel.  Every chunk of a
    // tensor of ordinary size is walked; of a huge one, the first and last thousand.
    const int64_t c_count = chunks_of(e.numel, chunk);
    int64_t covered = 0;
    for (int64_t c = 0; c < c_count; ++c) {
      if (c == 1000 && c_count > 4000) {
        c = c_count - 1000;
        covered = c * chunk;
      }
      for (int sub = 0; sub < kSub; ++sub) {
        const int64_t base = tile_base(e.first_chunk + c, sub, e.first_chunk, chunk, tile);
        const int64_t remain = e.numel - base;
        const int64_t count = remain <= 0 ? 0 : (remain < tile ? remain : tile);
        if (count > 0) {
          CHECK(base == covered, "tensor %d chunk %" PRId64 " sub %d starts at %" PRId64 ", expected %" PRId64, t, c, sub, base, covered);
          covered += count;
        }
      }
    }
    CHECK(covered == e.numel, "tensor %d: tiles cover %" PRId64 " of %" PRId64 " elements", t, covered, e.numel);
  }
  if (n_chunks <= (int64_t)1 << 22) {
    std::vector<int32_t> map((size_t)n_chunks + 1, -5);
    build_chunk_map(entries.data(), n_tensors, map.data());
    CHECK(map[(size_t)n_chunks] == -5, "chunk map written past its end");
    FewTable few;
    std::memset(&few, 0, sizeof(few));
    if (n_tensors <= kFew) {
      for (int t = 0; t < n_tensors; ++t) few.e[t] = entries[(size_t)t];
      finish_few(&few, n_tensors);
    }
    for (int64_t c = 0; c < n_chunks; ++c) {
      const int t = map[(size_t)c];
      CHECK(t >= 0 && t < n_tensors, "chunk %" PRId64 " maps to tensor %d", c, t);
      const TensorEntry& e = entries[(size_t)t];
      CHECK(e.first_chunk <= c && c < e.first_chunk + chunks_of(e.numel, entry_chunk_elems(e)), "chunk %" PRId64 " is outside tensor %d", c, t);
      if (n_tensors <= kFew && n_tensors > 0) CHECK(few_lookup(few, c) == t, "few_lookup(%" PRId64 ") = %d, map says %d", c, few_lookup(few, c), t);
    }
  }
}

static void check_rejections() {
  int64_t numel[2] = {16, 16};
  const void* a[2] = {(const void*)0x1000, (const void*)0x2000};
  const void* const* lists[2] = {a, a};
  TensorEntry out[2];
  int64_t n = 0;
  CHECK(build_entries(-1, lists, 2, 3, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_SIZE, "negative tensor count");
  CHECK(build_entries(2, lists, 2, 3, numel, nullptr, 9, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_DTYPE, "dtype");
  CHECK(build_entries(2, lists, 2, 3, nullptr, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_NULL, "null numel");
  const void* const* holes[2] = {a, nullptr};
  CHECK(build_entries(2, holes, 2, 3, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_NULL, "missing needed list");
  CHECK(build_entries(2, holes, 2, 1, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_OK, "an unneeded list may be null");
  int64_t both_empty[2] = {0, 0};
  CHECK(build_entries(2, holes, 2, 3, both_empty, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_OK && n == 0,
        "a needed list may be null when no tensor has elements");
  const void* b[2] = {(const void*)0x1000, nullptr};
  const void* const* with_null[2] = {a, b};
  CHECK(build_entries(2, with_null, 2, 3, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_NULL, "null buffer of a non-empty tensor");
  int64_t empty_second[2] = {16, 0};
  CHECK(build_entries(2, with_null, 2, 3, empty_second, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_OK, "null buffer of an empty tensor is fine");
  const void* odd[2] = {(const void*)0x1001, (const void*)0x2000};
  const void* const* misaligned[2] = {a, odd};
  CHECK(build_entries(2, misaligned, 2, 3, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_ALIGN, "element alignment");
  const void* two[2] = {(const void*)0x1002, (const void*)0x2000};
  const void* const* bf16_ok[2] = {a, two};
  CHECK(build_entries(2, bf16_ok, 2, 3, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_OK && !(out[0].flags & kEntryVec), "2-byte aligned bf16");
  CHECK(build_entries(2, bf16_ok, 2, 3, numel, nullptr, OPTIMI_F32, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_ALIGN, "2-byte aligned fp32");
  int64_t negative[2] = {16, -1};
  CHECK(build_entries(2, lists, 2, 3, negative, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_SIZE, "negative numel");
  int64_t huge[2] = {INT64_MAX, INT64_MAX};
  CHECK(build_entries(2, lists, 2, 3, huge, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_SIZE, "numel that would overflow");
  int64_t at_limit[2] = {kMaxChunks * chunk_elems(OPTIMI_BF16), 1};
  CHECK(build_entries(1, lists, 2, 3, at_limit, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_OK && n == kMaxChunks, "largest list");
  CHECK(build_entries(2, lists, 2, 3, at_limit, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_SIZE, "one chunk past the largest list");
  CHECK(build_entries(kMaxTensors + 1, lists, 2, 3, numel, nullptr, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_SIZE,
        "more tensors than one workgroup each can cover in a grid");
  CHECK(build_entries(0, nullptr, 0, 0, nullptr, nullptr, OPTIMI_F32, 0u, kMaxChunks, nullptr, &n) == OPTIMI_OK && n == 0, "empty list");
  // per-tensor dtypes: each is validated, and an array that only 16-bit tensors have may be absent for fp32 ones
  const int bad_dtypes[2] = {OPTIMI_BF16, 7};
  CHECK(build_entries(2, lists, 2, 3, numel, bad_dtypes, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_DTYPE, "per-tensor dtype");
  const int bf16_f32[2] = {OPTIMI_BF16, OPTIMI_F32};
  CHECK(build_entries(2, with_null, 2, 3, numel, bf16_f32, OPTIMI_BF16, 0u, kMaxChunks, out, &n) == OPTIMI_ERR_NULL, "null buffer of an fp32 tensor");
  CHECK(build_entries(2, with_null, 2, 3, numel, bf16_f32, OPTIMI_BF16, 2u, kMaxChunks, out, &n) == OPTIMI_OK && out[1].ptr[1] == nullptr &&
            (out[1].flags & kEntryF32) && !(out[0].flags & kEntryF32) && n == 2,
        "16-bit-only array of an fp32 tensor");
  const int f32_bf16[2] = {OPTIMI_F32, OPTIMI_BF16};
  CHECK(build_entries(2, with_null, 2, 3, numel, f32_bf16, OPTIMI_BF16, 2u, kMaxChunks, out, &n) == OPTIMI_ERR_NULL, "16-bit-only array of a 16-bit tensor");
}

int main(int argc, char** argv) {
  const int rounds = argc > 1 ? std::atoi(argv[1]) : 400;
  check_rejections();
  const int counts[] = {0, 1, 2, 3, 15, 16, 17, 40, 290};
  int lists = 0;
  for (int r = 0; r < rounds; ++r) {
    const int dtype = (int)(rng() % 3);
    const int n_arrays = 4 + (int)(rng() % 4);
    const uint32_t need = (uint32_t)(rng() % (1u << n_arrays)) | 1u;
    check_list(counts[rng() % 9], dtype, n_arrays, need, false);
    check_list(counts[rng() % 9], 1 + (int)(rng() % 2), n_arrays, need | bit(n_arrays - 1), false, true);
    lists += 2;
  }
  check_list(100000, OPTIMI_BF16, 5, 0x1f, true, true);
  ++lists;
  for (int dtype = 0; dtype < 3; ++dtype) {  // 100,000 small tensors, as a gradient-release stress list has them
    check_list(100000, dtype, 5, 0x1f, true);
    ++lists;
  }
  std::printf("table_fuzz ok: %d lists\n", lists);
  return 0;
}
