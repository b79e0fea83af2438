#include "common.hpp"
using namespace sq;
extern "C" size_t sq_kmeans_workspace_bytes(int64_t, int64_t, int64_t, int64_t) { return 0; }
extern "C" int sq_kmeans_train(const DLTensor*, DLTensor*, DLTensor*, DLTensor*, DLTensor*, int32_t, void*) {
  SQ_FAIL(SQ_EUNSUPPORTED, "sq_kmeans_train: not built yet");
}
extern "C" int sq_reverse_index(const DLTensor*, DLTensor*, DLTensor*, DLTensor*, void*) {
  SQ_FAIL(SQ_EUNSUPPORTED, "sq_reverse_index: not built yet");
}
extern "C" int sq_index_add(const DLTensor*, const DLTensor*, DLTensor*, DLTensor*, void*) {
  SQ_FAIL(SQ_EUNSUPPORTED, "sq_index_add: not built yet");
}
extern "C" int sq_topk_select(const DLTensor*, const DLTensor*, const DLTensor*, const DLTensor*, DLTensor*, DLTensor*,
                              int32_t, void*) {
  SQ_FAIL(SQ_EUNSUPPORTED, "sq_topk_select: not built yet");
}
