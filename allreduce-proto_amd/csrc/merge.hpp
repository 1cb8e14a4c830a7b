// Merging the launches of different emulated ranks while a whole-world allreduce is recorded.
//
// A recorded world is one ordered chain of launches on one stream (see capi.hip).  In that chain the
// launches the ranks issue for one step of the algorithm are independent of one another -- they
// are what N devices would run side by side -- yet each pays a kernel boundary of its own: 8 ranks
// x 14 steps = 112 launches where 14 would do.  While a world is being recorded, every rank
// therefore hands its launch to this collector instead of the stream.  The collector keeps one
// pending launch of adds and one of copies and appends the segments of each new launch to them;
// it puts a pending launch on the stream only when it must:
//
//   * a segment of the new launch reads memory that a pending segment writes, or writes memory
//     that a pending segment reads or writes (then the pending launch has to run first: that is
//     the order in which they were issued, and segments of one launch run concurrently);
//   * the pending launch would exceed the kernel's segment table, or would write more bytes than
//     the limit its owner has set (the kernels choose their store policy by the bytes a launch
//     writes, and a merged launch should stay on the side of that choice its parts were on);
//   * something else is about to use the stream (a device copy, the end of the recording).
//
// The rule looks at memory only, not at the protocol: every ordering the engine relies on between
// two launches on one in-order stream is there because the later one touches memory the earlier
// one touches, so keeping the issue order between exactly those pairs keeps every result, bit for
// bit.  All segments pending at any moment are mutually independent by construction, so the order
// in which the two pending launches are put on the stream does not matter.
//
// Only recordings of whole worlds use this.  A rank replayed alone keeps its chain: its launches
// touch disjoint memory, and the chain is what stands for its dependency on the other ranks there.
#pragma once

#include <stdint.h>

#include "segments.hpp"
#include "status.hpp"

namespace ibcomm_hip {

template <class B>
class LaunchCollector {
 public:
  using Stream = typename B::Stream;

  // Takes one launch as the engine would have issued it on `s`.
  int Add(const SegmentBatch& batch, int dtype, Stream s) {
    SegmentBatch in;  // without the empty segments: their pointers may be anything
    in.count = 0;
    for (int i = 0; i < batch.count; i++)
      if (batch.seg[i].n != 0) in.seg[in.count++] = batch.seg[i];
    collected_++;
    if (in.count == 0) return kOk;
    const size_t es = DTypeSize(dtype);
    if (es == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
    // one stream and one element type at a time
    if ((add_.count || copy_.count) && (!(s == stream_) || dtype != dtype_)) IBCOMM_RETURN_IF_ERROR(Flush());
    stream_ = s;
    dtype_ = dtype;
    const bool is_add = in.seg[0].b != nullptr;
    SegmentBatch& mine = is_add ? add_ : copy_;
    SegmentBatch& other = is_add ? copy_ : add_;
    uint64_t in_bytes = 0;
    for (int i = 0; i < in.count; i++) in_bytes += in.seg[i].n * es;
    uint64_t& mine_bytes = is_add ? add_bytes_ : copy_bytes_;
    if (Conflicts(in, other, es)) IBCOMM_RETURN_IF_ERROR(FlushOne(&other));
    if (mine.count + in.count > kMaxSegments || (mine.count && mine_bytes + in_bytes > write_limit_) || Conflicts(in, mine, es))
      IBCOMM_RETURN_IF_ERROR(FlushOne(&mine));
    for (int i = 0; i < in.count; i++) mine.seg[mine.count++] = in.seg[i];
    mine_bytes += in_bytes;
    return kOk;
  }

  // A merged launch writes at most this many bytes (a launch that is larger on its own stays as it is).
  void set_write_limit(uint64_t bytes) { write_limit_ = bytes; }

  // Puts everything pending on the stream.
  int Flush() {
    IBCOMM_RETURN_IF_ERROR(FlushOne(&add_));
    return FlushOne(&copy_);
  }

  // Forgets what is pending (a recording that failed).
  void Discard() {
    add_.count = copy_.count = 0;
    add_bytes_ = copy_bytes_ = 0;
  }

  uint64_t collected() const { return collected_; }  // launches handed in
  uint64_t issued() const { return issued_; }        // launches put on the stream
  void ResetCounters() { collected_ = issued_ = 0; }

 private:
  static bool Overlaps(const void* p, uint64_t pb, const void* q, uint64_t qb) {
    const char* a = static_cast<const char*>(p);
    const char* b = static_cast<const char*>(q);
    return a < b + qb && b < a + pb;
  }
  // Does any segment of `in` have to run after some segment of `pending`?
  static bool Conflicts(const SegmentBatch& in, const SegmentBatch& pending, size_t es) {
    for (int i = 0; i < in.count; i++) {
      const Segment& n = in.seg[i];
      const uint64_t nb = n.n * es;
      for (int j = 0; j < pending.count; j++) {
        const Segment& p = pending.seg[j];
        const uint64_t pb = p.n * es;
        // written by both, or written by the new one and read by the pending one
        if (Overlaps(n.dst, nb, p.dst, pb) || Overlaps(n.dst, nb, p.a, pb) || (p.b && Overlaps(n.dst, nb, p.b, pb))) return true;
        // read by the new one and written by the pending one
        if (Overlaps(n.a, nb, p.dst, pb) || (n.b && Overlaps(n.b, nb, p.dst, pb))) return true;
      }
    }
    return false;
  }
  int FlushOne(SegmentBatch* pending) {
    if (pending->count == 0) return kOk;
    const int rc = B::LaunchSegments(*pending, dtype_, stream_, 0);
    pending->count = 0;
    (pending == &add_ ? add_bytes_ : copy_bytes_) = 0;
    issued_++;
    return rc;
  }

  SegmentBatch add_{}, copy_{};
  uint64_t add_bytes_ = 0, copy_bytes_ = 0;  // bytes the pending launches write
  uint64_t write_limit_ = UINT64_MAX;
  Stream stream_{};
  int dtype_ = kF32;
  uint64_t collected_ = 0, issued_ = 0;
};

}  // namespace ibcomm_hip
