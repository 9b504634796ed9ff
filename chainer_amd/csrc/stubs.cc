// Entry points that are declared but not implemented yet report NotImplementedError.
#include "common.h"
using namespace hipcx;
#define STUB(name) return Guard([&] { throw Error(HIPCX_NOT_IMPLEMENTED_ERROR, #name " is not implemented"); })
extern "C" {
size_t hipcx_reduce_workspace_size(const hipcx_array*, const int8_t*, int, const hipcx_array*) { return 0; }
int hipcx_sum(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_sum); }
int hipcx_amax(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_amax); }
int hipcx_argmax(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_argmax); }
size_t hipcx_dot_workspace_size(const hipcx_array*, const hipcx_array*, const hipcx_array*) { return 0; }
int hipcx_dot(const hipcx_array*, const hipcx_array*, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_dot); }
size_t hipcx_conv_workspace_size(const hipcx_array*, const hipcx_array*, const hipcx_array*) { return 0; }
int hipcx_conv(const hipcx_array*, const hipcx_array*, const hipcx_array*, const int64_t*, const int64_t*, int, const hipcx_array*,
               void*, size_t, void*) { STUB(hipcx_conv); }
int hipcx_fixed_batch_norm(const hipcx_array*, const hipcx_array*, const hipcx_array*, const hipcx_array*, const hipcx_array*,
                           hipcx_scalar, const int8_t*, int, const hipcx_array*, void*) { STUB(hipcx_fixed_batch_norm); }
int hipcx_max_pool(const hipcx_array*, const int64_t*, const int64_t*, const int64_t*, int, const hipcx_array*, void*) { STUB(hipcx_max_pool); }
int hipcx_average_pool(const hipcx_array*, const int64_t*, const int64_t*, const int64_t*, int, const hipcx_array*, void*) { STUB(hipcx_average_pool); }
int hipcx_take(const hipcx_array*, const hipcx_array*, int8_t, const hipcx_array*, int, int32_t*, void*) { STUB(hipcx_take); }
}
