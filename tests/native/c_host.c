/* A plain C program against include/sideaware.h: what a C maintainer of the reference's callers
 * (example_llmc_rope.cu:137-144) would write.  It needs no GPU: it registers op headers, checks
 * that the same text gives the same id, and compiles one for gfx950. */
#include <stdio.h>
#include <string.h>

#include "../../include/sideaware.h"

static const char *FILL =
    "typedef int o0;\n"
    "struct unused {};\n"
    "typedef unused o1, o2, o3, i0, i1, i2, i3;\n"
    "constexpr bool reverse_order = false;\n"
    "constexpr bool input_evict[4] = {0,0,0,0};\n"
    "__device__ void elementwise_op(size_t element_idx, int sideband,\n"
    "                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,\n"
    "                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {\n"
    "    out0 = sideband;\n"
    "}\n";

int main(void) {
    char log[4096];
    int a, b;
    if (sideaware_create_kernel(NULL) != 0 || sideaware_create_kernel("") != 0) return 1;
    a = sideaware_create_kernel(FILL);
    b = sideaware_create_kernel_advanced(FILL, false, 2);
    if (a < 1 || a != b) return 2;
    if (sideaware_compile_check(FILL, 0, log, sizeof log) != 0) { fprintf(stderr, "%s\n", log); return 3; }
    if (sideaware_compile_check("this is not an op header", 0, log, sizeof log) == 0) return 4;
    if (strstr(log, "error") == NULL) return 5;
    /* calls that must return at once without a device */
    sideaware_memcpy(NULL, NULL, 0, 0, NULL);
    sideaware_free_auto(NULL, 0, 0, NULL);
    sideaware_compression(true);
    sideaware_prealloc_config(1, 10);
    if (strlen(sideaware_kernel_source()) < 1000) return 6;
    printf("c host ok: kernel id %d\n", a);
    return 0;
}
