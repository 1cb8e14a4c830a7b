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

// An expression compiled once into a postfix program and evaluated per element on a small stack.
class Expr {
 public:
  explicit Expr(const std::string& text) : s_(text) {
    Sum();
    Skip();
    if (pos_ != s_.size()) ok_ = false;
  }
  bool ok() const { return ok_; }
  double Eval(const Vars& v) const {
    double st[64];
    int top = 0;
    for (const Ins& in : prog_) {
      switch (in.op) {
        case kNum: st[top++] = in.value; break;
        case kP: st[top++] = v.p; break;
        case kNp: st[top++] = v.np; break;
        case kN: st[top++] = v.n; break;
        case kNb: st[top++] = v.nb; break;
        case kI: st[top++] = v.i; break;
        case kNeg: st[top - 1] = -st[top - 1]; break;
        case kAdd: top--; st[top - 1] += st[top]; break;
        case kSub: top--; st[top - 1] -= st[top]; break;
        case kMul: top--; st[top - 1] *= st[top]; break;
        case kDiv: top--; st[top - 1] /= st[top]; break;
      }
    }
    return top == 1 ? st[0] : 0.0;
  }

 private:
  enum Op { kNum, kP, kNp, kN, kNb, kI, kNeg, kAdd, kSub, kMul, kDiv };
  struct Ins {
    Op op;
    double value;
  };
  void Emit(Op op, double value = 0) {
    prog_.push_back(Ins{op, value});
    if (op <= kI) {
      if (++depth_ > 60) ok_ = false;
    } else if (op != kNeg) {
      depth_--;
    }
  }
  void Skip() {
    while (pos_ < s_.size() && isspace(static_cast<unsigned char>(s_[pos_]))) pos_++;
  }
  bool Eat(char c) {
    Skip();
    if (pos_ < s_.size() && s_[pos_] == c) {
      pos_++;
      return true;
    }
    return false;
  }
  void Sum() {
    Product();
    for (;;) {
      if (Eat('+')) { Product(); Emit(kAdd); }
      else if (Eat('-')) { Product(); Emit(kSub); }
      else return;
    }
  }
  void Product() {
    Unary();
    for (;;) {
      if (Eat('*')) { Unary(); Emit(kMul); }
      else if (Eat('/')) { Unary(); Emit(kDiv); }
      else return;
    }
  }
  void Unary() {
    if (Eat('-')) { Unary(); Emit(kNeg); return; }
    if (Eat('+')) { Unary(); return; }
    Atom();
  }
  void Atom() {
    Skip();
    if (pos_ >= s_.size()) { ok_ = false; Emit(kNum, 0); return; }
    if (s_[pos_] == '(') {
      pos_++;
      Sum();
      if (!Eat(')')) ok_ = false;
      return;
    }
    if (isdigit(static_cast<unsigned char>(s_[pos_])) || s_[pos_] == '.') {
      char* end = nullptr;
      const double a = strtod(s_.c_str() + pos_, &end);
      pos_ = static_cast<size_t>(end - s_.c_str());
      Emit(kNum, a);
      return;
    }
    if (isalpha(static_cast<unsigned char>(s_[pos_]))) {
      const size_t b = pos_;
      while (pos_ < s_.size() && isalnum(static_cast<unsigned char>(s_[pos_]))) pos_++;
      const std::string name = s_.substr(b, pos_ - b);
      if (name == "p") return Emit(kP);
      if (name == "np") return Emit(kNp);
      if (name == "n") return Emit(kN);
      if (name == "nb") return Emit(kNb);
      if (name == "i") return Emit(kI);
    }
    ok_ = false;
    Emit(kNum, 0);
  }
  std::string s_;
  size_t pos_ = 0;
  bool ok_ = true;
  int depth_ = 0;
  std::vector<Ins> prog_;
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
      util::EndProcess(util::IBCOMM_ERROR_CODE::CUDA_ERROR);                                   \
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
  for (const std::string& e : {init_expr, check_expr}) {
    if (!Expr(e).ok()) {
      fprintf(stderr, "Invalid expression: '%s'\n", e.c_str());
      return 1;
    }
  }

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
      const Expr init(init_expr);
      for (size_t i = 0; i < n; i++) {
        v.i = static_cast<double>(i);
        host[i] = static_cast<ElemType>(init.Eval(v));
      }
      ElemType *send = nullptr, *recv = nullptr;
      HIP_OR_EXIT(hipMalloc(&send, n * sizeof(ElemType)));
      HIP_OR_EXIT(hipMalloc(&recv, n * sizeof(ElemType)));
      HIP_OR_EXIT(hipMemcpy(send, host.data(), n * sizeof(ElemType), hipMemcpyHostToDevice));
      if (algorithm == "ring") comms[r]->AllreduceRingCuda(send, recv, n);
      else comms[r]->AllreduceRabenseifnerCuda(send, recv, n);
      HIP_OR_EXIT(hipMemcpy(host.data(), recv, n * sizeof(ElemType), hipMemcpyDeviceToHost));
      const Expr check(check_expr);
      size_t reported = 0;
      for (size_t i = 0; i < n; i++) {
        v.i = static_cast<double>(i);
        const double want = check.Eval(v);
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
