// Static communication plans of the two allreduce algorithms for one rank.
//
// The reference drives each algorithm with a polling state machine whose
// queues are filled up front (AllreduceRingCuda: reg_q / first_send_q,
// ibcomm/allreduce_cuda_impl.h:61-89; AllreduceRabenseifnerCuda: recv_q /
// send_q / first_send_q, :387-466).  What those queues fix -- and what a peer
// running the reference would rely on -- is, per ordered pair of ranks, the
// order of chunks on the wire, plus which chunks are reduced and which are only
// stored.  A Plan states exactly that as two lists, so that the executor can
// issue it as stream-ordered device work instead of polling:
//
//   recvs[k]  the k-th message this rank consumes: from whom, which chunk, and
//             what happens to it (added to the rank's own contribution, added
//             to the running partial sum, or stored as a finished result);
//   sends[k]  the k-th message this rank emits: to whom, which chunk, and the
//             receive whose result it forwards (-1: straight from sendbuf).
//
// Both lists are in the order the reference's queues hold them.
#pragma once

#include <vector>

#include "partition.hpp"

namespace ibcomm_hip {

enum Algo : int { kRing = 0, kRabenseifner = 1 };

enum RecvKind : int {
  kReduceWithSendbuf = 0,  // recvbuf[c] = incoming + sendbuf[c]
  kReduceAccumulate = 1,   // recvbuf[c] = incoming + recvbuf[c]
  kGather = 2,             // recvbuf[c] = incoming (finished sum)
};

struct RecvOp {
  int chunk;
  int peer;
  int kind;
};

struct SendOp {
  int chunk;
  int peer;
  int dep;  // index into Plan::recvs of the op that produces the data, -1 = data is sendbuf[chunk]
};

struct Plan {
  int algo = kRing;
  int world_size = 1;
  int rank = 0;
  Partition part;
  std::vector<RecvOp> recvs;
  std::vector<SendOp> sends;
  // Per receive: the one send that forwards its result when that result is needed nowhere else on
  // this rank (a later gather overwrites the chunk), else -1.  Such a partial sum may be produced
  // straight into send staging instead of recvbuf.
  std::vector<int> forward_only;
};

namespace detail {

inline void MarkForwardOnly(Plan* plan) {
  const size_t n = plan->recvs.size();
  plan->forward_only.assign(n, -1);
  std::vector<int> sends_of(n, 0), send_index(n, -1);
  for (size_t k = 0; k < plan->sends.size(); k++) {
    const int d = plan->sends[k].dep;
    if (d >= 0) {
      sends_of[d]++;
      send_index[d] = static_cast<int>(k);
    }
  }
  std::vector<char> gathered_later(plan->part.ranges.size(), 0);
  for (size_t j = n; j-- > 0;) {
    const RecvOp& r = plan->recvs[j];
    if (r.kind == kGather) {
      gathered_later[r.chunk] = 1;
    } else if (gathered_later[r.chunk] && sends_of[j] == 1) {
      plan->forward_only[j] = send_index[j];
    }
  }
}

}  // namespace detail

namespace detail {

inline void PushGroupDescending(const Partition& p, int g, std::vector<int>* out) {
  for (int c = p.group_back(g); c >= p.group_first[g]; c--) out->push_back(c);
}

}  // namespace detail

// Ring (allreduce_cuda_impl.h:53-99, 137-157).  Rank r receives from r-1 and
// sends to r+1.  Reduce-scatter consumes groups r-1, r-2, ..., r+1, allgather
// consumes groups r, r-1, ..., r+2; inside a group chunk ids descend.  On the
// wire rank r first emits its own group from sendbuf, then every chunk it
// reduced (the last reduced group, r+1, is the first allgather hop), then every
// gathered chunk except those of group r+2, whose next hop would be its origin.
inline void BuildRingPlan(int world_size, int rank, Plan* plan) {
  const Partition& p = plan->part;
  const int N = world_size, r = rank;
  const int from = (r - 1 + N) % N, to = (r + 1) % N;
  plan->recvs.clear();
  plan->sends.clear();
  std::vector<int> ids;
  detail::PushGroupDescending(p, r, &ids);
  for (int c : ids) plan->sends.push_back(SendOp{c, to, -1});
  for (int i = 0; i < N - 1; i++) {
    ids.clear();
    detail::PushGroupDescending(p, (r - i - 1 + N) % N, &ids);
    for (int c : ids) {
      plan->recvs.push_back(RecvOp{c, from, kReduceWithSendbuf});
      plan->sends.push_back(SendOp{c, to, static_cast<int>(plan->recvs.size()) - 1});
    }
  }
  const int final_group = (r + 2) % N;
  for (int i = 0; i < N - 1; i++) {
    const int g = (r - i + N) % N;
    ids.clear();
    detail::PushGroupDescending(p, g, &ids);
    for (int c : ids) {
      plan->recvs.push_back(RecvOp{c, from, kGather});
      if (g != final_group) plan->sends.push_back(SendOp{c, to, static_cast<int>(plan->recvs.size()) - 1});
    }
  }
}

// Rabenseifner (allreduce_cuda_impl.h:387-466).  Halving step s pairs r with
// r ^ (1 << s); the lower rank of a pair keeps the back half of its current
// window of groups and sends the front half, the higher rank the opposite.
// Doubling step s pairs r with r ^ (1 << (k-1-s)) and exchanges whole windows.
// Chunk ids ascend inside every window.  Step-0 sends go out from sendbuf;
// every later send forwards what the most recent receive on that chunk left in
// recvbuf.  The reference first copies sendbuf to recvbuf (:332-333) and then
// adds in place; here the step-0 reduction reads sendbuf directly, which is the
// same sum, and every other element of recvbuf is overwritten by a later
// gather, so that copy is not needed.
inline void BuildRabenseifnerPlan(int world_size, int rank, Plan* plan) {
  const Partition& p = plan->part;
  const int N = world_size, r = rank;
  const int k = GetExpOfTwo(N);
  plan->recvs.clear();
  plan->sends.clear();
  std::vector<int> last_writer(p.ranges.size(), -1);
  std::vector<SendOp> later_sends;  // send_q; step-0 sends (first_send_q) go out ahead of it

  int start = 0, end = N;
  for (int step = 0; step < k; step++) {
    const int peer = r ^ (1 << step);
    int ss, se, rs, re;
    if (r < peer) { ss = start; se = end - (end - start) / 2; rs = se; re = end; }
    else          { rs = start; re = end - (end - start) / 2; ss = re; se = end; }
    // sends of this step read what earlier steps produced, so resolve them before this step's receives
    for (int g = ss; g < se; g++) {
      for (int c = p.group_first[g]; c <= p.group_back(g); c++) {
        if (step == 0) plan->sends.push_back(SendOp{c, peer, -1});
        else later_sends.push_back(SendOp{c, peer, last_writer[c]});
      }
    }
    for (int g = rs; g < re; g++) {
      for (int c = p.group_first[g]; c <= p.group_back(g); c++) {
        plan->recvs.push_back(RecvOp{c, peer, step == 0 ? kReduceWithSendbuf : kReduceAccumulate});
        last_writer[c] = static_cast<int>(plan->recvs.size()) - 1;
      }
    }
    start = rs;
    end = re;
  }
  for (int step = 0; step < k; step++) {
    const int peer = r ^ (1 << (k - step - 1));
    const int ss = start, se = end;
    int rs, re;
    if (r > peer) { rs = se; re = rs + (end - start); }
    else          { re = ss; rs = re - (end - start); }
    for (int g = ss; g < se; g++)
      for (int c = p.group_first[g]; c <= p.group_back(g); c++) later_sends.push_back(SendOp{c, peer, last_writer[c]});
    for (int g = rs; g < re; g++) {
      for (int c = p.group_first[g]; c <= p.group_back(g); c++) {
        plan->recvs.push_back(RecvOp{c, peer, kGather});
        last_writer[c] = static_cast<int>(plan->recvs.size()) - 1;
      }
    }
    start = ss < rs ? ss : rs;
    end = se > re ? se : re;
  }
  plan->sends.insert(plan->sends.end(), later_sends.begin(), later_sends.end());
}

// Validates the call the way the reference does and fills *plan.  world_size 1
// yields an empty plan (the caller copies).  Error order follows the
// reference: Rabenseifner checks the process count before it partitions
// (:342-354).
inline int BuildPlan(int algo, int world_size, int rank, size_t len_elements, size_t sizeof_element,
                     const char* env_chunksize, Plan* plan) {
  plan->algo = algo;
  plan->world_size = world_size;
  plan->rank = rank;
  plan->recvs.clear();
  plan->sends.clear();
  if (world_size < 1 || rank < 0 || rank >= world_size) return Fail(kInvalidArgument, "rank %d outside world of %d", rank, world_size);
  plan->forward_only.clear();
  if (world_size == 1) {
    plan->part = Partition();
    return kOk;
  }
  if (algo == kRabenseifner && GetExpOfTwo(world_size) == 0) {
    return Fail(kNotSupported, "Currently, rabenseifner's algorithm doesn't support non-power-of-2 processes.");
  }
  IBCOMM_RETURN_IF_ERROR(BuildPartition(len_elements, sizeof_element, world_size, env_chunksize, &plan->part));
  if (algo == kRing) BuildRingPlan(world_size, rank, plan);
  else if (algo == kRabenseifner) BuildRabenseifnerPlan(world_size, rank, plan);
  else return Fail(kInvalidArgument, "unknown algorithm %d", algo);
  detail::MarkForwardOnly(plan);
  return kOk;
}

}  // namespace ibcomm_hip
