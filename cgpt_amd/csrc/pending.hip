// Entry points whose kernels are not written yet: they report that clearly
// instead of leaving the symbol out of the library.
#include "common.hpp"

extern "C" int cgptx_cut_cross_entropy_forward_backward(float*, void*, void*, const void*, const void*,
                                                        const uint32_t*, size_t, size_t, size_t, float, int, int,
                                                        cgptx_stream) {
    return cgptx::fail(CGPTX_RUNTIME, "cut_cross_entropy_forward_backward: not implemented yet");
}
extern "C" int cgptx_flash_gqa_attention_backward_with_lse(void*, void*, void*, const void*, const void*,
                                                           const float*, const void*, const void*, const void*,
                                                           size_t, size_t, size_t, size_t, size_t, size_t, float, int,
                                                           size_t, int, int, cgptx_stream) {
    return cgptx::fail(CGPTX_RUNTIME, "flash_gqa_attention_backward_with_lse: not implemented yet");
}
extern "C" int cgptx_flash_gqa_attention_backward(void*, void*, void*, const void*, const void*, const void*,
                                                  const void*, size_t, size_t, size_t, size_t, size_t, size_t, float,
                                                  int, size_t, int, int, cgptx_stream) {
    return cgptx::fail(CGPTX_RUNTIME, "flash_gqa_attention_backward: not implemented yet");
}
extern "C" int cgptx_flash_gqa_attention_forward(void*, float*, const void*, const void*, const void*, size_t, size_t,
                                                 size_t, size_t, size_t, size_t, float, int, size_t, int,
                                                 cgptx_stream) {
    return cgptx::fail(CGPTX_RUNTIME, "flash_gqa_attention_forward: not implemented yet");
}
