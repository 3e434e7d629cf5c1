// Host-side tables of a list launch: argument validation, the tensor table, the chunk map, and
// the index arithmetic a workgroup uses to find its tile.  Plain C++ with no HIP call, so that
// a CPU build (with sanitizers) can exercise exactly the code the library runs; the functions
// the kernels share are marked OPTIMI_HD.
//
// A list of tensors is cut into chunks of kChunkBytes per array (so a chunk of an fp32 tensor
// holds half the elements of a chunk of a 16-bit one); chunks are numbered through the whole
// list, tensor after tensor, and kSub workgroups share a chunk.  A workgroup learns
// which tensor its chunk belongs to either from a chunk map in device memory (large lists) or,
// for lists of at most kFew tensors, by searching a table that travels as a kernel argument.
// This takes the place of the per-tensor Python launch loops of the reference
// (optimi/adam.py:551-583, lion.py:470-492, stableadamw.py:689-725, adan.py:679-711).

#ifndef OPTIMI_TABLES_H
#define OPTIMI_TABLES_H

#include <climits>
#include <cstdint>
#include <cstring>

#include "optimi_hip.h"

#if defined(__HIPCC__)
#define OPTIMI_HD __host__ __device__ __forceinline__
#else
#define OPTIMI_HD inline
#endif

namespace optimi_tables {

constexpr int kMaxArrays = 7;       // Adan: p g m diff sq prev kahan
constexpr int kChunkBytes = 16384;  // bytes per array per chunk: the granule of the chunk map
constexpr int kFew = 16;            // lists up to this long travel as a kernel argument

struct TensorEntry {
  void* ptr[kMaxArrays];
  int64_t numel;
  int64_t first_chunk;  // index of this tensor's first chunk within the launch
  uint32_t flags;       // kEntry* bits
  uint32_t pad;
};
constexpr uint32_t kEntryVec = 1;     // all buffers 16-byte aligned: the vector path applies
constexpr uint32_t kEntryCached = 2;  // read full tiles with ordinary cached loads instead of streaming ones
constexpr uint32_t kEntryF32 = 4;     // the tensor is fp32 (a list may mix fp32 tensors with tensors of one 16-bit dtype)
static_assert(sizeof(TensorEntry) == 80, "TensorEntry layout");

struct FewTable {
  TensorEntry e[kFew];
  int32_t first_chunk[kFew];  // e[t].first_chunk again, packed so that one scalar load fetches all; INT32_MAX from n on
  int32_t n;
  int32_t pad;
};

constexpr uint32_t bit(int i) { return 1u << i; }

// One workgroup of 1024 threads per tensor must fit a grid of fewer than 2^32 threads
// (StableAdamW's per-tensor reduction).
constexpr int kMaxTensors = (1 << 22) - 1;

inline bool valid_dtype(int dtype) { return dtype == OPTIMI_F32 || dtype == OPTIMI_BF16 || dtype == OPTIMI_F16; }
inline int elem_bytes(int dtype) { return dtype == OPTIMI_F32 ? 4 : 2; }
inline int64_t chunk_elems(int dtype) { return kChunkBytes / elem_bytes(dtype); }
inline int64_t chunks_of(int64_t numel, int64_t chunk) { return (numel + chunk - 1) / chunk; }

inline int64_t entry_chunk_elems(const TensorEntry& e) { return kChunkBytes / ((e.flags & kEntryF32) ? 4 : 2); }

// Validates a list and writes one entry per tensor.  `lists[a]` may be nullptr for an array the
// launch does not touch (`need` has its bit clear) or that only tensors without elements would use.  `dtypes`, when not null, gives every
// tensor's own dtype (a mixed list); otherwise all tensors have `dtype`.  Arrays in
// `low_precision_only` (the Kahan buffer) exist for 16-bit tensors only: an fp32 tensor's
// pointer there is ignored.  `max_chunks` bounds the list (chunk numbers are kept in 32-bit
// tables).  Returns an optimi_status.
inline int build_entries(int n_tensors, const void* const* const* lists, int n_arrays, uint32_t need, const int64_t* numel,
                         const int* dtypes, int dtype, uint32_t low_precision_only, int64_t max_chunks, TensorEntry* out,
                         int64_t* n_chunks_out) {
  if (n_tensors < 0 || n_tensors > kMaxTensors) return OPTIMI_ERR_SIZE;
  if (!dtypes && !valid_dtype(dtype)) return OPTIMI_ERR_DTYPE;
  if (n_arrays < 0 || n_arrays > kMaxArrays) return OPTIMI_ERR_SIZE;
  if (n_tensors > 0 && (!numel || !out)) return OPTIMI_ERR_NULL;
  int64_t n_chunks = 0;
  for (int t = 0; t < n_tensors; ++t) {
    const int dt = dtypes ? dtypes[t] : dtype;
    if (!valid_dtype(dt)) return OPTIMI_ERR_DTYPE;
    const int64_t chunk = chunk_elems(dt);
    const uintptr_t eb = (uintptr_t)elem_bytes(dt);
    TensorEntry& e = out[t];
    std::memset(&e, 0, sizeof(e));
    if (numel[t] < 0) return OPTIMI_ERR_SIZE;
    if (numel[t] > max_chunks * chunk) return OPTIMI_ERR_SIZE;  // also keeps the sums below from overflowing
    e.numel = numel[t];
    e.first_chunk = n_chunks;
    e.flags = kEntryVec | (dt == OPTIMI_F32 ? kEntryF32 : 0u);
    for (int a = 0; a < n_arrays; ++a) {
      if (!(need & bit(a))) continue;
      if (dt == OPTIMI_F32 && (low_precision_only & bit(a))) continue;
      const void* p = (lists && lists[a]) ? lists[a][t] : nullptr;  // a missing list is a list of null pointers
      if (!p && numel[t] > 0) return OPTIMI_ERR_NULL;
      const uintptr_t u = (uintptr_t)p;
      if (u % eb) return OPTIMI_ERR_ALIGN;
      if (u % 16) e.flags &= ~kEntryVec;
      e.ptr[a] = const_cast<void*>(p);
    }
    n_chunks += chunks_of(numel[t], chunk);
    if (n_chunks > max_chunks) return OPTIMI_ERR_SIZE;
  }
  if (n_chunks_out) *n_chunks_out = n_chunks;
  return OPTIMI_OK;
}

// chunk -> tensor for every chunk of the launch; `map` has room for the launch's chunk count.
inline void build_chunk_map(const TensorEntry* entries, int n_tensors, int32_t* map) {
  for (int t = 0; t < n_tensors; ++t) {
    const int64_t c0 = entries[t].first_chunk, c1 = c0 + chunks_of(entries[t].numel, entry_chunk_elems(entries[t]));
    for (int64_t c = c0; c < c1; ++c) map[c] = t;
  }
}

// Fills the packed search keys of a short list from its entries.
inline void finish_few(FewTable* few, int n_tensors) {
  few->n = n_tensors;
  for (int t = 0; t < kFew; ++t)
    few->first_chunk[t] = t < n_tensors ? (int32_t)few->e[t].first_chunk : INT32_MAX;
}

// The tensor that owns chunk `chunk_id` of a short list: the last one whose first chunk is not
// beyond it, i.e. the count of such tensors minus one - sixteen compares on one 64-byte load, no
// branches.  (A tensor without elements owns no chunk: it shares its first_chunk with its
// successor, which is later in the table and wins; trailing ones start past the last chunk.)
OPTIMI_HD int few_lookup(const FewTable& few, int64_t chunk_id) {
  // first_chunk[t] <= chunk_id  <=>  first_chunk[t] - chunk_id - 1 < 0; both are below 2^31 / 16,
  // so the difference cannot wrap and its sign bit is the comparison (plain integer arithmetic
  // keeps the whole search in scalar registers)
  const int32_t c = (int32_t)chunk_id;
  uint32_t count = 0;
  for (int t = 0; t < kFew; ++t) count += (uint32_t)(few.first_chunk[t] - c - 1) >> 31;
  return (int)count - 1;
}

// First element, within its tensor, of the tile that workgroup `sub` of chunk `chunk_id` covers.
// The tile is [base, base + tile) cut off at the tensor's numel; base >= numel means no work.
OPTIMI_HD int64_t tile_base(int64_t chunk_id, int sub, int64_t first_chunk, int64_t chunk, int64_t tile) {
  return (chunk_id - first_chunk) * chunk + (int64_t)sub * tile;
}

}  // namespace optimi_tables

#endif  // OPTIMI_TABLES_H
