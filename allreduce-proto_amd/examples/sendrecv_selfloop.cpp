// Point-to-point messaging through a communicator whose queue pairs are connected to each other.
//
// The reference's tests/sendrecv_test.cpp brings up ONE IBVerbsCommunicator of world size 2,
// connects its queue pair for peer 1 to its queue pair for peer 0 (CreateQueuePair(1),
// RegisterProcess(0, ...), RegisterQueuePair(1, ...)) and then sends "to 0" what it receives
// "from 1".  This program drives the drop-in class the same way, over more sizes and both
// directions of the wire, with host and device buffers, and also checks the rule that a second
// non-blocking send to a peer needs the first one's SendWait (ibverbs_communicator.cpp:375-378),
// which ends the process with status 4.
//
//   sendrecv_selfloop            exit status 0 if every message arrived intact
//   sendrecv_selfloop twice      posts two non-blocking sends in a row: exit status 4
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <vector>

#include "ibcomm/ibverbs_communicator.h"

namespace {

int failures = 0;

void Expect(bool ok, const char* what, size_t n) {
  if (ok) return;
  failures++;
  fprintf(stderr, "FAILED: %s (%zu bytes)\n", what, n);
}

// One message of n bytes sent on queue pair `to`, received on the pair wired to it.
void PingHost(IBVerbsCommunicator* comm, int to, int from, size_t n, unsigned char seed) {
  std::vector<unsigned char> out(n), in(n, 0xee);
  for (size_t i = 0; i < n; i++) out[i] = static_cast<unsigned char>(seed + i * 7);
  comm->Send(to, out.data(), n, false);
  comm->Recv(from, in.data(), n);  // blocking
  comm->SendWait(to);
  Expect(memcmp(out.data(), in.data(), n) == 0, "host message", n);
}

void PingDevice(IBVerbsCommunicator* comm, int to, int from, size_t n) {
  std::vector<unsigned char> out(n), back(n, 0);
  for (size_t i = 0; i < n; i++) out[i] = static_cast<unsigned char>(i * 13 + 5);
  void *src = nullptr, *dst = nullptr;
  if (hipMalloc(&src, n) != hipSuccess || hipMalloc(&dst, n) != hipSuccess) {
    Expect(false, "hipMalloc", n);
    return;
  }
  Expect(hipMemcpy(src, out.data(), n, hipMemcpyHostToDevice) == hipSuccess, "upload", n);
  comm->Recv(from, dst, n, false);
  comm->Send(to, src, n, false);
  comm->RecvWait(from);
  comm->SendWait(to);
  Expect(hipMemcpy(back.data(), dst, n, hipMemcpyDeviceToHost) == hipSuccess, "download", n);
  Expect(out == back, "device message", n);
  (void)hipFree(src);
  (void)hipFree(dst);
}

}  // namespace

int main(int argc, char** argv) {
  IBVerbsCommunicator comm(2);
  const ProcessInfo pair1 = comm.CreateQueuePair(1);
  const ProcessInfo pair0 = comm.RegisterProcess(0, pair1);
  comm.RegisterQueuePair(1, pair0);

  if (argc > 1 && strcmp(argv[1], "twice") == 0) {
    int a = 1, b = 2;
    comm.Send(0, &a, sizeof a, false);
    comm.Send(0, &b, sizeof b, false);  // NOT_SUPPORTED: SendWait must come first
    return 0;                           // not reached
  }

  // the reference's own sequence: an int to 0, received from 1, twice
  int value = 10, value2 = -1;
  comm.Send(0, &value, sizeof value, false);
  comm.Recv(1, &value2, sizeof value2);
  comm.SendWait(0);
  Expect(value2 == 10, "first int", sizeof value);
  value2 = -1;
  comm.Send(0, &value2, sizeof value, false);
  comm.Recv(1, &value, sizeof value2);
  comm.SendWait(0);
  Expect(value == -1, "second int", sizeof value);

  const size_t sizes[] = {1, 3, 64, 4097, 1 << 20};
  unsigned char seed = 1;
  for (size_t n : sizes) {
    PingHost(&comm, 0, 1, n, seed++);  // sent to 0, arrives from 1
    PingHost(&comm, 1, 0, n, seed++);  // and the other way along the same wire
    PingDevice(&comm, 0, 1, n);
  }
  // polling forms: nothing to receive yet, then a message, then its completion
  Expect(!comm.RecvPoll(1), "RecvPoll with nothing posted", 0);
  int x = 77, y = 0;
  comm.Recv(1, &y, sizeof y, false);
  Expect(!comm.RecvPoll(1), "RecvPoll before the send", sizeof y);
  comm.Send(0, &x, sizeof x, false);
  while (!comm.RecvPoll(1)) {
  }
  while (!comm.SendPoll(0)) {
  }
  Expect(y == 77, "polled int", sizeof y);

  printf(failures ? "sendrecv_selfloop: %d failures\n" : "sendrecv_selfloop: OK\n", failures);
  return failures ? 10 : 0;
}
