// One translation unit per (element type, head dim); the build passes
// -DFA2_T=BF16|FP16 -DFA2_TAG=bf16|fp16 -DFA2_D=64|128|256.
#include "fa2_fwd_kernel.hpp"

#define FA2_CAT3(a, b, c) a##b##_##c
#define FA2_NAME(tag, d) FA2_CAT3(launch_fwd_, tag, d)

namespace fa2 {
hipError_t FA2_NAME(FA2_TAG, FA2_D)(bool bias, bool drop, KArgs& a, hipStream_t s) {
	return launch_fwd_t<FA2_T, FA2_D>(bias, drop, a, s);
}
}  // namespace fa2
