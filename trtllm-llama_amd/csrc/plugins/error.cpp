// Thread-local error text behind tllm_last_error(): every entry point of the C ABI returns a code and leaves its reason here.
// A translation unit of its own so that both libraries (the plugin library and the stack engine) carry it.
#include "../kernels/kernels.h"
#include <cstdarg>
#include <cstdio>

namespace tllm
{

static thread_local char g_err[2048] = {0};

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

const char* last_error()
{
    return g_err;
}

} // namespace tllm

extern "C" const char* tllm_last_error(void)
{
    return tllm::last_error();
}
