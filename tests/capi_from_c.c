/* The header compiles as plain C and the library is usable from a C program with no Python or torch in the
 * process: loads it, checks a few host-only entry points and an argument check.  Built and run by
 * tests/test_capi_cpu.py; prints "ok" on success. */
#include <dlfcn.h>
#include <stdio.h>
#include <string.h>

#include "bsa_mi355x.h"

int main(int argc, char** argv) {
    if (argc < 2) return 2;
    void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
    if (!lib) { fprintf(stderr, "dlopen: %s\n", dlerror()); return 3; }
    int (*version)(void) = (int (*)(void))dlsym(lib, "bsa_version");
    int (*num_selected)(double, int) = (int (*)(double, int))dlsym(lib, "bsa_num_selected");
    size_t (*workspace_bytes)(const bsa_3d_params*) = (size_t (*)(const bsa_3d_params*))dlsym(lib, "bsa_workspace_bytes");
    const char* (*last_error)(void) = (const char* (*)(void))dlsym(lib, "bsa_last_error");
    int (*fwd)(const void*, const void*, const void*, const int32_t*, const int32_t*, const uint64_t*, void*, float*, int, int,
               int64_t, int64_t, int, int, int, int, float, int, void*) =
        (int (*)(const void*, const void*, const void*, const int32_t*, const int32_t*, const uint64_t*, void*, float*, int, int,
                 int64_t, int64_t, int, int, int, int, float, int, void*))dlsym(lib, "bsa_fwd");
    if (!version || !num_selected || !workspace_bytes || !last_error || !fwd) return 4;
    if (version() < 100) return 5;
    if (num_selected(0.9375, 1440) != 90 || num_selected(0.9, 10) != 0) return 6;
    bsa_3d_params p;
    memset(&p, 0, sizeof(p));
    p.B = 1; p.Hn = 32; p.D = 128; p.dtype = BSA_BF16;
    p.Tq = p.Tk = 24; p.Hq = p.Hk = 45; p.Wq = p.Wk = 80;
    p.tq = p.hq = p.wq = p.tk = p.hk = p.wk = 4;
    p.k_sel = 90; p.sm_scale = 0.088388f; p.cdf_threshold = 0.f;
    const size_t ws = workspace_bytes(&p);
    if (ws < (size_t)1 << 30 || ws > (size_t)2 << 30) return 7;        /* k and v in fragment order (1.5 GB) + a few hundred MB at 720p */
    p.D = 96;
    if (workspace_bytes(&p) != 0) return 8;                            /* unsupported head dim: 0 and an error text */
    if (strlen(last_error()) == 0) return 9;
    if (fwd(NULL, NULL, NULL, NULL, NULL, NULL, NULL, NULL, 1, 1, 64, 64, 128, 64, 64, 1, 0.1f, BSA_BF16, NULL) != BSA_ERR_BAD_ARG)
        return 10;
    printf("ok %zu\n", ws);
    dlclose(lib);
    return 0;
}
