// errors.hip -- the error slot of the C ABI (errors.h) and the ABI version: the one source every build of the library contains.
#include "hw.h"
#include "errors.h"

static thread_local char g_err[512] = "";

void exl2_set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" {

const char* exl2_last_error(void) { return g_err; }

int exl2_abi_version(void) { return 1; }

}
