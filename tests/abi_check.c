/* The C side of the boundary: include/evoattn.h compiles as plain C99, the library loads with
 * dlopen and exports every entry point, and the host-side validation returns the documented
 * codes.  No GPU is touched: every call below is rejected before a launch.
 * Built and run by tests/test_abi.py::test_header_is_plain_c_and_the_library_loads_from_c. */
#include <dlfcn.h>
#include <stdio.h>
#include <string.h>

#include "evoattn.h"

typedef int (*version_fn)(void);
typedef const char *(*strerror_fn)(int);
typedef int (*check_fn)(const EvoAttnParams *, int);
typedef size_t (*bytes_fn)(const EvoAttnParams *);
typedef int (*run_fn)(const EvoAttnParams *, void *);
typedef const char *(*name_fn)(const EvoAttnParams *, int);

#define NEED(cond, what) do { if (!(cond)) { fprintf(stderr, "abi_check: %s\n", what); return 1; } } while (0)

int main(int argc, char **argv) {
    void *lib;
    version_fn version;
    strerror_fn strerr;
    check_fn check;
    bytes_fn prep_bytes, ws_bytes;
    run_fn fwd, fwd_static, bwd;
    name_fn path, kernels;
    EvoAttnParams p;
    static char fake[64];

    NEED(argc == 2, "usage: abi_check <path to libevoattn.so>");
    lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
    NEED(lib != NULL, dlerror());
    *(void **)&version = dlsym(lib, "evoattn_version");
    *(void **)&strerr = dlsym(lib, "evoattn_strerror");
    *(void **)&check = dlsym(lib, "evoattn_check");
    *(void **)&prep_bytes = dlsym(lib, "evoattn_prep_bytes");
    *(void **)&ws_bytes = dlsym(lib, "evoattn_bwd_workspace_bytes");
    *(void **)&fwd = dlsym(lib, "evoattn_fwd");
    *(void **)&fwd_static = dlsym(lib, "evoattn_fwd_static");
    *(void **)&bwd = dlsym(lib, "evoattn_bwd");
    *(void **)&path = dlsym(lib, "evoattn_path");
    *(void **)&kernels = dlsym(lib, "evoattn_kernels");
    NEED(version && strerr && check && prep_bytes && ws_bytes && fwd && fwd_static && bwd && path && kernels, "missing export");
    NEED(version() == EVOATTN_VERSION, "version mismatch between header and library");

    memset(&p, 0, sizeof p);
    NEED(check(NULL, EVO_PASS_FWD) == EVO_EINVAL, "NULL block accepted");
    NEED(check(&p, EVO_PASS_FWD) == EVO_EINVAL, "zero sizes accepted");
    p.B = 1; p.S = 4; p.N = 64; p.H = 2; p.D = 32;
    p.dtype = EVO_BF16; p.bias_dtype = EVO_NONE; p.mask_kind = EVO_MASK_NONE;
    p.scale = 0.17677669f;
    p.stride_b = 4 * 64 * 2 * 32; p.stride_h = 4 * 64 * 32; p.stride_s = 64 * 32; p.stride_n = 32;
    p.q = p.k = p.v = fake; p.o = fake; p.lse = (float *)fake;
    NEED(check(&p, EVO_PASS_FWD) == EVO_OK, "valid forward block rejected");
    NEED(strcmp(path(&p, EVO_PASS_FWD), "mfma") == 0, "bf16 head dim 32 not on the matrix-core path");
    NEED(prep_bytes(&p) > 0 && prep_bytes(&p) <= EVOATTN_STATIC_PREP_BYTES, "prep size");
    NEED(fwd(&p, NULL) == EVO_EWORKSPACE, "forward without a prep buffer accepted");
    NEED(check(&p, EVO_PASS_BWD) == EVO_EINVAL, "backward without gradients accepted");
    p.dout = fake; p.dq = p.dk = p.dv = fake;
    NEED(check(&p, EVO_PASS_BWD) == EVO_EWORKSPACE, "backward without a workspace accepted");
    NEED(ws_bytes(&p) >= (size_t)(1 * 2 * 4 * 64) * 4, "workspace smaller than delta");
    p.flags = 0x40;                                    /* a bit the header does not declare */
    NEED(check(&p, EVO_PASS_FWD) == EVO_EINVAL && fwd_static(&p, NULL) == EVO_EINVAL && bwd(&p, NULL) == EVO_EINVAL,
         "undeclared flag accepted");
    p.flags = 0;
    p.D = 24;
    NEED(check(&p, EVO_PASS_FWD) == EVO_EUNSUPPORTED, "head dim 24 accepted by the C ABI");
    NEED(strlen(strerr(EVO_EUNSUPPORTED)) > 0 && strlen(strerr(EVO_EALIGN)) > 0, "error strings");
    p.D = 32;
    NEED(strstr(kernels(&p, EVO_PASS_FWD), "mfma_fwd") != NULL, "kernel names");
    printf("abi_check ok: version %d, sizeof(EvoAttnParams) = %u\n", version(), (unsigned)sizeof(EvoAttnParams));
    dlclose(lib);
    return 0;
}
