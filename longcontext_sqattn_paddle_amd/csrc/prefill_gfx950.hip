#include "common.hpp"
using namespace sq;
extern "C" size_t sq_prefill_workspace_bytes(int64_t, int64_t, int64_t, int64_t) { return 0; }
extern "C" int sq_prefill_fwd(const DLTensor*, const DLTensor*, const DLTensor*, const DLTensor*, const DLTensor*,
                              DLTensor*, DLTensor*, DLTensor*, const sq_prefill_params*, void*) {
  SQ_FAIL(SQ_EUNSUPPORTED, "sq_prefill_fwd: not built yet");
}
