// Thin extern "C" view of the reference's own ibcomm/util.h, compiled where it
// lies (-I<reference root>) into oracle/_ref/.  TEST INFRASTRUCTURE ONLY: it
// lets the tests check the oracle's restatement of ceilDiv and GetExpOfTwo
// against the reference's code itself.  util.h is the only reference file
// that builds without InfiniBand Verbs, CUDA or MPI headers.
#include "ibcomm/util.h"

extern "C" {
long long ref_ceil_div(long long a, long long b) { return util::ceilDiv<long long>(a, b); }
int ref_get_exp_of_two(int n) { return util::GetExpOfTwo(n); }
int ref_error_code(int which) {
  switch (which) {
    case 0: return static_cast<int>(util::IBCOMM_ERROR_CODE::INVALID_ARGUMENT);
    case 1: return static_cast<int>(util::IBCOMM_ERROR_CODE::IBVERBS_ERROR);
    case 2: return static_cast<int>(util::IBCOMM_ERROR_CODE::CUDA_ERROR);
    case 3: return static_cast<int>(util::IBCOMM_ERROR_CODE::NOT_SUPPORTED);
  }
  return -1;
}
}
