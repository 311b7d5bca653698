// Grouped expert GEMM (placeholder until the MFMA kernel lands).
#include "common.hpp"

using namespace brt;

extern "C" int brt_hip_grouped_gemm(const void* x, const void* const* weights,
                                    const void* const* biases, void* out, const int32_t* loads,
                                    int E, int P, int K, int N, int act, void* stream) {
  return fail(BRT_E_UNSUPPORTED, "grouped GEMM is not built yet");
}
