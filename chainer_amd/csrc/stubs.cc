// Entry points that are declared but not implemented yet report NotImplementedError.
#include "common.h"
using namespace hipcx;
#define STUB(name) return Guard([&] { throw Error(HIPCX_NOT_IMPLEMENTED_ERROR, #name " is not implemented"); })
extern "C" {
size_t hipcx_reduce_workspace_size(const hipcx_array*, const int8_t*, int, const hipcx_array*) { return 0; }
int hipcx_sum(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_sum); }
int hipcx_amax(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_amax); }
int hipcx_argmax(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*) { STUB(hipcx_argmax); }
int hipcx_take(const hipcx_array*, const hipcx_array*, int8_t, const hipcx_array*, int, int32_t*, void*) { STUB(hipcx_take); }
}
