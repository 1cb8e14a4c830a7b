// Staging memory and streams for the chunk pipelines, resident in HBM.
//
// Role of the reference's MemoryPool / MemoryController / MemoryBlock / Memory
// (ibcomm/memory_pool.h:28-283, memory_pool.cpp:11-55): pre-allocated blocks
// carved into chunk-sized slots that incoming messages land in, plus the pool
// of streams the per-chunk work is issued on, both handed out first-in
// first-out.  Differences that come from living on one MI355X:
//
//   * blocks are device memory (hipMalloc), not pinned host memory registered
//     with an HCA; nothing crosses PCIe;
//   * a slot is handed back as soon as the kernel that reads it has been
//     *enqueued*, together with the event that marks that kernel's completion;
//     the next user of the slot orders itself after that event on the device.
//     The host never waits for a slot, so a handful of slots sustain the whole
//     pipeline; returned slots are reused before untouched ones, so those few
//     slots are also all the memory a collective's staging ever writes.  The
//     engine never grows the pool in the middle of a collective as long as its
//     blocks hold one slot: when every slot is taken it launches what it has
//     collected (which hands the landing slots back) or, for send staging,
//     leaves the partial sum in recvbuf; getMemory() itself still grows the
//     pool on exhaustion, as the reference's does (memory_pool.h:229-231);
//   * slots are carved on demand, so a block of tiny chunks costs nothing for
//     the slots nobody asks for and no cap on their number is needed;
//   * each slot keeps 16 spare bytes so that a message can land at the same
//     16-byte phase as the recvbuf range it will be added to, which keeps the
//     kernel's body on dwordx4 accesses for odd chunk offsets;
//   * carving uses every slot that fits ((i + 1) * stride <= block) where the
//     reference's strict '<' (memory_pool.h:269) leaves the last one unused,
//     and a chunk larger than a block makes the pool allocate a block that
//     fits two chunks instead of handing out memory it does not have
//     (memory_pool.h:229-233);
//   * IBCOMM_MEMORY_POOL_PRE_ALLOC is read as a 64-bit value without the
//     reference's 1 GiB ceiling (memory_pool.h:163), default 256 MiB;
//     IBCOMM_NUM_CUDA_STREAM keeps its name and its (0, 1024] range
//     (memory_pool.h:139-154); streams are created on first use and the
//     default is 8, because a process drives 4 hardware queues on this GPU.
#pragma once

#include <stdlib.h>

#include <deque>
#include <memory>
#include <vector>

#include "status.hpp"

namespace ibcomm_hip {

template <class B>
struct Memory {
  char* base = nullptr;            // 256-byte aligned start of the slot
  size_t capacity = 0;             // usable bytes including the phase margin
  typename B::Event free_event{};  // valid iff has_free_event: last reader's completion
  bool has_free_event = false;
  typename B::Stream free_stream{};  // stream free_event was recorded on
  // Where a message bound for `target` should land so that both share their 16-byte phase.
  char* LandingFor(const void* target) const { return base + (reinterpret_cast<uintptr_t>(target) & 15); }
};

template <class B>
class MemoryPool;

template <class B>
class MemoryController {
 public:
  MemoryController() = default;
  MemoryController(const MemoryController&) = delete;
  MemoryController& operator=(const MemoryController&) = delete;
  ~MemoryController() { Release(); }

  bool active() const { return pool_ != nullptr; }
  // Slots the pool's blocks hold at this chunk size, handed out yet or not.
  size_t slot_count() const { return capacity_; }
  // Slots that can be handed out without growing the pool.
  size_t available() const { return vacant_.size() + (capacity_ - carved_); }
  int held() const { return held_; }
  int high_water() const { return high_water_; }

  // Hand-out (memory_pool.h:222-236): the slot that came back longest ago, else one that has never
  // been used, else the pool grows by one block.  Preferring returned slots keeps the memory a
  // collective writes to as small as its pipeline depth (a handful of slots) however large the
  // block is; on MI355X that working set then lives in the 256 MB memory-side cache, and a ring
  // step's stores into it run measurably faster than stores that walk through the whole block
  // (config 2: 205 -> 196 us per rank schedule).
  int getMemory(Memory<B>** out);
  // The same without growth: false (and *out untouched) when every slot is taken.
  bool TryGetMemory(Memory<B>** out);
  // FIFO return (memory_pool.h:238-242); `after` completes when the slot's contents are dead.
  void returnMemory(Memory<B>* m, typename B::Event after, typename B::Stream stream) {
    m->free_event = after;
    m->free_stream = stream;
    m->has_free_event = true;
    vacant_.push_back(m);
    held_--;
  }
  void returnMemory(Memory<B>* m) {
    vacant_.push_back(m);
    held_--;
  }
  void Release();

 private:
  friend class MemoryPool<B>;
  struct Block {
    char* base;
    size_t slots;  // block bytes / stride
  };
  void AddBlock(char* block, size_t block_bytes) {
    blocks_.push_back(Block{block, block_bytes / stride_});
    capacity_ += blocks_.back().slots;
  }
  Memory<B>* CarveNext();

  MemoryPool<B>* pool_ = nullptr;
  size_t stride_ = 0;
  bool descending_ = false;
  std::vector<Block> blocks_;      // the pool's blocks as this chunk size divides them
  size_t capacity_ = 0;            // slots in all blocks
  size_t carved_ = 0;              // of which handed out at least once, block after block, in the hand-out direction
  size_t carve_block_ = 0, carve_slot_ = 0;  // the next untouched slot
  std::vector<std::unique_ptr<Memory<B>>> slots_;  // one object per slot handed out so far
  std::deque<Memory<B>*> vacant_;  // returned, oldest first
  int held_ = 0;
  int high_water_ = 0;
};

template <class B>
class MemoryPool {
 public:
  static constexpr int kDefaultNumStreams = 8;
  static constexpr size_t kDefaultPreAlloc = size_t(256) << 20;

  MemoryPool() = default;
  MemoryPool(const MemoryPool&) = delete;
  MemoryPool& operator=(const MemoryPool&) = delete;
  ~MemoryPool() { Destroy(); }

  // Reads the knobs and allocates the first block (memory_pool.h:86-100).  A non-zero
  // `block_bytes` replaces IBCOMM_MEMORY_POOL_PRE_ALLOC (for a backend whose memory is bounded).
  int Init(size_t block_bytes = 0) {
    IBCOMM_RETURN_IF_ERROR(ReadNumStreams(&max_streams_));
    IBCOMM_RETURN_IF_ERROR(ReadPreAlloc(&block_bytes_));
    if (block_bytes) block_bytes_ = block_bytes;
    return AllocateBlock(block_bytes_, nullptr);
  }

  void Destroy() {
    for (auto s : streams_) B::StreamDestroy(s);
    streams_.clear();
    for (auto& b : blocks_) B::Free(b.first);
    blocks_.clear();
  }

  // One controller at a time (memory_pool.h:111-121).
  // With phase_margin every slot keeps 16 spare bytes (see Memory::LandingFor); without, slots of a
  // chunk size that is a multiple of 256 bytes are contiguous.  Slots are first handed out from the
  // lowest address upwards, or with `descending` from the highest downwards.
  int GetController(size_t chunk_bytes, bool phase_margin, bool descending, MemoryController<B>* c) {
    if (controller_in_use_) return Fail(kNotSupported, "Currently, MemoryController is in use.");
    if (chunk_bytes == 0) return Fail(kInvalidArgument, "chunk size must be positive");
    controller_in_use_ = true;
    c->pool_ = this;
    c->stride_ = (chunk_bytes + (phase_margin ? 16 : 0) + 255) & ~size_t(255);
    c->descending_ = descending;
    c->slots_.clear();
    c->vacant_.clear();
    c->blocks_.clear();
    c->capacity_ = c->carved_ = c->carve_block_ = c->carve_slot_ = 0;
    c->held_ = 0;
    c->high_water_ = 0;
    for (auto& b : blocks_) c->AddBlock(b.first, b.second);
    return kOk;
  }

  // While set, NextStream() hands out this one stream only.  Used to record a collective as a
  // single ordered chain of device work (a HIP graph without cross-stream edges).
  void OverrideStream(typename B::Stream s) {
    override_ = s;
    has_override_ = true;
  }
  void ClearOverride() { has_override_ = false; }
  bool has_override() const { return has_override_; }

  // Round-robin over at most max_streams() streams, created on first use.
  int NextStream(typename B::Stream* out) {
    if (has_override_) {
      *out = override_;
      return kOk;
    }
    if (static_cast<int>(streams_.size()) < max_streams_ && cursor_ >= streams_.size()) {
      typename B::Stream s;
      IBCOMM_RETURN_IF_ERROR(B::StreamCreate(&s));
      streams_.push_back(s);
    }
    if (cursor_ >= streams_.size()) cursor_ = 0;
    *out = streams_[cursor_++];
    return kOk;
  }
  void RewindStreams() { cursor_ = 0; }

  int SynchronizeStreams() {
    for (auto s : streams_) IBCOMM_RETURN_IF_ERROR(B::StreamSynchronize(s));
    return kOk;
  }

  int max_streams() const { return max_streams_; }
  size_t streams_created() const { return streams_.size(); }
  const std::vector<typename B::Stream>& streams() const { return streams_; }
  size_t block_bytes() const { return block_bytes_; }
  size_t blocks() const { return blocks_.size(); }
  size_t bytes_allocated() const {
    size_t t = 0;
    for (auto& b : blocks_) t += b.second;
    return t;
  }

 private:
  friend class MemoryController<B>;

  static int ReadNumStreams(int* out) {
    const char* v = getenv("IBCOMM_NUM_CUDA_STREAM");
    if (!v) {
      *out = kDefaultNumStreams;
      return kOk;
    }
    const int n = atoi(v);
    if (n <= 0 || n > 1024) return Fail(kInvalidArgument, "Invalid value for IBCOMM_NUM_CUDA_STREAM: %s", v);
    *out = n;
    return kOk;
  }

  static int ReadPreAlloc(size_t* out) {
    const char* v = getenv("IBCOMM_MEMORY_POOL_PRE_ALLOC");
    if (!v) {
      *out = kDefaultPreAlloc;
      return kOk;
    }
    const long long n = atoll(v);
    if (n < 4) return Fail(kInvalidArgument, "Invalid value for IBCOMM_MEMORY_POOL_PRE_ALLOC: %s", v);
    *out = static_cast<size_t>(n);
    return kOk;
  }

  int AllocateBlock(size_t bytes, char** out) {
    void* p = nullptr;
    IBCOMM_RETURN_IF_ERROR(B::Malloc(&p, bytes));
    blocks_.emplace_back(static_cast<char*>(p), bytes);
    if (out) *out = static_cast<char*>(p);
    return kOk;
  }

  void CompleteMemoryController() { controller_in_use_ = false; }

  int max_streams_ = kDefaultNumStreams;
  size_t block_bytes_ = kDefaultPreAlloc;
  std::vector<std::pair<char*, size_t>> blocks_;
  std::vector<typename B::Stream> streams_;
  size_t cursor_ = 0;
  bool controller_in_use_ = false;
  typename B::Stream override_{};
  bool has_override_ = false;
};

// The next slot nobody has used yet: blocks in the order they were allocated, inside a block from the
// lowest address upwards or, descending, from the highest downwards.
template <class B>
Memory<B>* MemoryController<B>::CarveNext() {
  while (carve_block_ < blocks_.size() && carve_slot_ == blocks_[carve_block_].slots) {
    carve_block_++;
    carve_slot_ = 0;
  }
  if (carve_block_ == blocks_.size()) return nullptr;
  const Block& b = blocks_[carve_block_];
  const size_t i = descending_ ? b.slots - 1 - carve_slot_ : carve_slot_;
  carve_slot_++;
  carved_++;
  slots_.emplace_back(new Memory<B>());
  Memory<B>* m = slots_.back().get();
  m->base = b.base + i * stride_;
  m->capacity = stride_;
  return m;
}

template <class B>
bool MemoryController<B>::TryGetMemory(Memory<B>** out) {
  if (!pool_) return false;
  Memory<B>* m = nullptr;
  if (!vacant_.empty()) {
    m = vacant_.front();
    vacant_.pop_front();
  } else {
    m = CarveNext();
  }
  if (!m) return false;
  held_++;
  if (held_ > high_water_) high_water_ = held_;
  *out = m;
  return true;
}

template <class B>
int MemoryController<B>::getMemory(Memory<B>** out) {
  if (!pool_) return Fail(kInvalidArgument, "MemoryController is not attached to a pool");
  if (TryGetMemory(out)) return kOk;
  size_t bytes = pool_->block_bytes();
  if (bytes < 2 * stride_) bytes = 2 * stride_;
  char* block = nullptr;
  IBCOMM_RETURN_IF_ERROR(pool_->AllocateBlock(bytes, &block));
  AddBlock(block, bytes);
  return TryGetMemory(out) ? kOk : Fail(kDeviceError, "a new pool block of %zu bytes holds no slot of %zu", bytes, stride_);
}

template <class B>
void MemoryController<B>::Release() {
  if (!pool_) return;
  slots_.clear();
  vacant_.clear();
  blocks_.clear();
  capacity_ = carved_ = carve_block_ = carve_slot_ = 0;
  pool_->CompleteMemoryController();
  pool_ = nullptr;
}

}  // namespace ibcomm_hip
