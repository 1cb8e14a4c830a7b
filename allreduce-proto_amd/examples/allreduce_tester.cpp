// Loopback counterpart of PFNProto's integration tester (ibcomm/allreduce_tester.cpp).
//
//   allreduce_tester <np> <algorithm> <buffer size> <init expr> <check expr>
//
// The reference is started as `mpiexec -np <np> allreduce_tester <algorithm> ...`
// (tests/allreduce_test.py:91); here the <np> ranks are threads of one process that share the GPU,
// each with its own IBVerbsCommunicator.  Everything else follows the reference: element type int
// (:416), the buffer is filled element by element from <init expr> and compared with <check expr>
// after the allreduce (:290-322, eps 1e-12), variables p, np, n, nb, i (:18-27), size suffixes
// k/m/g (:205-238), exit status = number of ranks whose check failed (:396-405) or the library's
// error code.  Expressions: numbers, the five variables, + - * / and parentheses, which covers
// every expression the reference's tests use.
#include <hip/hip_runtime.h>

#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>
#include <thread>
#include <vector>

#include "ibcomm/ibverbs_communicator.h"

namespace {

struct Vars {
  double p, np, n, nb, i;
};

class Expr {
 public:
  explicit Expr(const std::string& text) : s_(text) {}
  bool Eval(const Vars& v, double* out) {
    v_ = &v;
    pos_ = 0;
    ok_ = true;
    const double r = Sum();
    Skip();
    if (pos_ != s_.size()) ok_ = false;
    *out = r;
    return ok_;
  }

 private:
  void Skip() {
    while (pos_ < s_.size() && isspace(static_cast<unsigned char>(s_[pos_]))) pos_++;
  }
  double Sum() {
    double a = Product();
    for (;;) {
      Skip();
      if (pos_ < s_.size() && s_[pos_] == '+') { pos_++; a += Product(); }
      else if (pos_ < s_.size() && s_[pos_] == '-') { pos_++; a -= Product(); }
      else return a;
    }
  }
  double Product() {
    double a = Unary();
    for (;;) {
      Skip();
      if (pos_ < s_.size() && s_[pos_] == '*') { pos_++; a *= Unary(); }
      else if (pos_ < s_.size() && s_[pos_] == '/') { pos_++; a /= Unary(); }
      else return a;
    }
  }
  double Unary() {
    Skip();
    if (pos_ < s_.size() && s_[pos_] == '-') { pos_++; return -Unary(); }
    if (pos_ < s_.size() && s_[pos_] == '+') { pos_++; return Unary(); }
    return Atom();
  }
  double Atom() {
    Skip();
    if (pos_ >= s_.size()) { ok_ = false; return 0; }
    if (s_[pos_] == '(') {
      pos_++;
      const double a = Sum();
      Skip();
      if (pos_ < s_.size() && s_[pos_] == ')') pos_++;
      else ok_ = false;
      return a;
    }
    if (isdigit(static_cast<unsigned char>(s_[pos_])) || s_[pos_] == '.') {
      char* end = nullptr;
      const double a = strtod(s_.c_str() + pos_, &end);
      pos_ = static_cast<size_t>(end - s_.c_str());
      return a;
    }
    if (isalpha(static_cast<unsigned char>(s_[pos_]))) {
      size_t b = pos_;
      while (pos_ < s_.size() && isalnum(static_cast<unsigned char>(s_[pos_]))) pos_++;
      const std::string name = s_.substr(b, pos_ - b);
      if (name == "p") return v_->p;
      if (name == "np") return v_->np;
      if (name == "n") return v_->n;
      if (name == "nb") return v_->nb;
      if (name == "i") return v_->i;
    }
    ok_ = false;
    return 0;
  }
  std::string s_;
  size_t pos_ = 0;
  bool ok_ = true;
  const Vars* v_ = nullptr;
};

bool ParseBytes(const char* src, size_t* out) {  // allreduce_tester.cpp:205-238
  size_t i = 0, n = 0;
  if (!isdigit(static_cast<unsigned char>(src[0]))) return false;
  while (isdigit(static_cast<unsigned char>(src[i]))) n = n * 10 + static_cast<size_t>(src[i++] - '0');
  switch (src[i]) {
    case 0: break;
    case 'k': case 'K': n *= 1024; break;
    case 'm': case 'M': n *= 1024 * 1024; break;
    case 'g': case 'G': n *= 1024ull * 1024 * 1024; break;
    default: return false;
  }
  *out = n;
  return true;
}

#define HIP_OR_EXIT(cmd)                                                                       \
  do {                                                                                         \
    hipError_t e_ = (cmd);                                                                     \
    if (e_ != hipSuccess) {                                                                    \
      fprintf(stderr, "%s failed: %s\n", #cmd, hipGetErrorString(e_));                         \
      exit(static_cast<int>(util::IBCOMM_ERROR_CODE::CUDA_ERROR));                             \
    }                                                                                          \
  } while (0)

}  // namespace

int main(int argc, char** argv) {
  using ElemType = int;
  if (argc != 6) {
    fprintf(stderr, "Usage: %s [np] [algorithm] [array size (Bytes)] [init expr] [check expr]\n", argv[0]);
    return 255;
  }
  const int np = atoi(argv[1]);
  const std::string algorithm = argv[2];
  size_t nbytes = 0;
  if (np < 1 || np > 1024) { fprintf(stderr, "np must be in [1, 1024]\n"); return 1; }
  if (algorithm != "ring" && algorithm != "rabenseifner") {
    fprintf(stderr, "Error: Unsupported algorithm %s\nSupported algorithms: ring, rabenseifner, \n", algorithm.c_str());
    return 1;
  }
  if (!ParseBytes(argv[3], &nbytes)) { fprintf(stderr, "Cannot parse an array size: '%s'\n", argv[3]); return 1; }
  if (nbytes < sizeof(ElemType)) {
    fprintf(stderr, "Warning: specified array size is smaller than the element size(%zu). Ceiling it up to %zu [bytes]\n",
            sizeof(ElemType), sizeof(ElemType));
    nbytes = sizeof(ElemType);
  }
  const size_t n = nbytes / sizeof(ElemType);
  const std::string init_expr = argv[4], check_expr = argv[5];

  HIP_OR_EXIT(hipSetDevice(0));
  std::vector<std::unique_ptr<IBVerbsCommunicator>> comms;
  for (int r = 0; r < np; r++) {
    comms.emplace_back(new IBVerbsCommunicator(np));
    for (int i = 0; i < np; i++) {  // same calls as the reference's bring-up; no-ops over the loopback
      if (i == r) continue;
      comms.back()->RegisterQueuePair(i, comms.back()->CreateQueuePair(i));
    }
    comms.back()->RegisterMyself(r);
  }

  std::vector<int> failed(np, 0);
  std::vector<std::thread> threads;
  for (int r = 0; r < np; r++) {
    threads.emplace_back([&, r]() {
      Vars v{static_cast<double>(r), static_cast<double>(np), static_cast<double>(n), static_cast<double>(nbytes), 0};
      std::vector<ElemType> host(n);
      Expr init(init_expr);
      for (size_t i = 0; i < n; i++) {
        v.i = static_cast<double>(i);
        double x;
        if (!init.Eval(v, &x)) { fprintf(stderr, "Invalid expression: '%s'\n", init_expr.c_str()); exit(1); }
        host[i] = static_cast<ElemType>(x);
      }
      ElemType *send = nullptr, *recv = nullptr;
      HIP_OR_EXIT(hipMalloc(&send, n * sizeof(ElemType)));
      HIP_OR_EXIT(hipMalloc(&recv, n * sizeof(ElemType)));
      HIP_OR_EXIT(hipMemcpy(send, host.data(), n * sizeof(ElemType), hipMemcpyHostToDevice));
      if (algorithm == "ring") comms[r]->AllreduceRingCuda(send, recv, n);
      else comms[r]->AllreduceRabenseifnerCuda(send, recv, n);
      HIP_OR_EXIT(hipMemcpy(host.data(), recv, n * sizeof(ElemType), hipMemcpyDeviceToHost));
      Expr check(check_expr);
      size_t reported = 0;
      for (size_t i = 0; i < n; i++) {
        v.i = static_cast<double>(i);
        double want;
        if (!check.Eval(v, &want)) { fprintf(stderr, "Invalid expression: '%s'\n", check_expr.c_str()); exit(1); }
        if (std::fabs(static_cast<double>(host[i]) - want) > 1e-12) {
          failed[r] = 1;
          if (reported++ < 10) fprintf(stderr, "[Rank %d] Error: Element [%zu] must be %g but actually is %d\n", r, i, want, host[i]);
        }
      }
      (void)hipFree(send);
      (void)hipFree(recv);
    });
  }
  for (auto& t : threads) t.join();
  int status = 0;
  for (int r = 0; r < np; r++) status += failed[r];
  comms.clear();
  return status;
}
