/* TEST INFRASTRUCTURE ONLY.  Opens oracle/_ref/libdecx_ref_cpu.so with lazy symbol
 * binding (Python's ctypes always binds eagerly) and hands back the address of the
 * C shim in it.  Lazy binding matters because the reference's NASM-only CPUID helper
 * is not part of that build; its symbol is never reached. */
#include <dlfcn.h>
#include <stddef.h>

void* ref_loader_sym(const char* lib_path, const char* symbol)
{
    void* h = dlopen(lib_path, RTLD_LAZY | RTLD_LOCAL);
    return h ? dlsym(h, symbol) : NULL;
}

const char* ref_loader_error(void) { return dlerror(); }
