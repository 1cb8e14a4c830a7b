// How an allreduce buffer is cut into chunks and how chunks are dealt to ranks.
//
// Same rule as IBVerbsCommunicator::SplitBuffer / GetRankToChunk
// (ibcomm/ibverbs_communicator.cpp:618-707): the chunk a given element falls
// in, and the rank group that chunk belongs to, decide the order in which the
// ranks' contributions are added, so this must agree with the reference
// element for element.  Pure integer host code.
//
// Deviation: offsets are kept in size_t.  The reference stores them in `int`
// (cpp:676-677) and is therefore limited to buffers below 2^31 elements; for
// every length it can handle the ranges are identical.
#pragma once

#include <stddef.h>
#include <stdlib.h>

#include <vector>

#include "status.hpp"

namespace ibcomm_hip {

struct Range {
  size_t begin;  // first element
  size_t end;    // one past the last element
  size_t size() const { return end - begin; }
};

struct Partition {
  std::vector<Range> ranges;     // chunk id -> element range
  std::vector<int> group_first;  // rank -> first chunk id of its group
  std::vector<int> group_count;  // rank -> number of chunks in its group
  int group_back(int rank) const { return group_first[rank] + group_count[rank] - 1; }
};

// util.h:151-154
template <typename T>
inline T CeilDiv(T a, T b) {
  return a % b ? a / b + 1 : a / b;
}

// util.h:156-175: log2(n) for powers of two, 0 otherwise (so also 0 for n == 1).
inline int GetExpOfTwo(int n) {
  if (n <= 0 || (n & (n - 1)) != 0) return 0;
  int p = 0;
  while ((1 << p) != n) p++;
  return p;
}

// IBCOMM_CHUNKSIZE as the reference reads it (cpp:619-634): getenv + atoi on
// every call; unset -> -1; a value <= 0 is an error.  `env` is the variable's
// text or nullptr.
inline int ParseChunkSize(const char* env, long* out_bytes) {
  if (env == nullptr) {
    *out_bytes = -1;
    return kOk;
  }
  const int v = atoi(env);
  if (v <= 0) return Fail(kInvalidArgument, "IBCOMM_CHUNKSIZE must be greater than 1");
  *out_bytes = v;
  return kOk;
}

inline int SplitBuffer(size_t len_elements, size_t sizeof_element, int world_size, const char* env_chunksize,
                       std::vector<Range>* out) {
  out->clear();
  if (len_elements < static_cast<size_t>(world_size)) {
    return Fail(kNotSupported,
                "Input vector is too short for current Allreduce algorithm.\n"
                "Incrase the number of the input vector to be larger than number of processes.\n");
  }
  long env_bytes = -1;
  IBCOMM_RETURN_IF_ERROR(ParseChunkSize(env_chunksize, &env_bytes));

  size_t chunks, per_chunk;
  if (env_bytes != -1) {
    if (static_cast<size_t>(env_bytes) % sizeof_element != 0) {
      return Fail(kInvalidArgument, "Selected `IBCOMM_CHUNKSIZE` is not divisible by `sizeof(T)`.");
    }
    per_chunk = static_cast<size_t>(env_bytes) / sizeof_element;
    chunks = CeilDiv(len_elements, per_chunk);
    if (chunks < 2 * static_cast<size_t>(world_size)) {
      return Fail(kInvalidArgument,
                  "Selected `IBCOMM_CHUNKSIZE` is too large.\n"
                  "Satisfy 2 * `world_size` <= `allreduce_bufsize` / `IBCOMM_CHUNKSIZE`.");
    }
  } else {
    chunks = 4 * static_cast<size_t>(world_size);
    per_chunk = CeilDiv(len_elements, chunks);
  }
  out->reserve(chunks);
  for (size_t i = 0; i < chunks; i++) {
    const size_t b = per_chunk * i;
    size_t e = per_chunk * (i + 1);
    if (e > len_elements) e = len_elements;
    if (b < e) out->push_back(Range{b, e});  // empty trailing chunks are dropped (cpp:679)
  }
  return kOk;
}

inline void GetRankToChunk(size_t n_ranges, int world_size, std::vector<int>* first, std::vector<int>* count) {
  first->assign(world_size, 0);
  count->assign(world_size, 0);
  const int per = static_cast<int>(n_ranges / world_size);
  const int rem = static_cast<int>(n_ranges % world_size);
  int id = 0;
  for (int r = 0; r < world_size; r++) {
    (*first)[r] = id;
    (*count)[r] = per + (r < rem ? 1 : 0);
    id += (*count)[r];
  }
}

inline int BuildPartition(size_t len_elements, size_t sizeof_element, int world_size, const char* env_chunksize,
                          Partition* p) {
  IBCOMM_RETURN_IF_ERROR(SplitBuffer(len_elements, sizeof_element, world_size, env_chunksize, &p->ranges));
  GetRankToChunk(p->ranges.size(), world_size, &p->group_first, &p->group_count);
  return kOk;
}

}  // namespace ibcomm_hip
