/*
 * yvex-rocm: the two inspection commands of the ROCm backend arm as a program of their own,
 * with the reference's command paths and exit codes:
 *
 *     yvex-rocm inspect backend rocm       context, bundle and exact primitive capabilities
 *     yvex-rocm inspect rocm [bandwidth]   device facts, or the bounded bandwidth fixture
 *
 * Inside the reference these are two rows of its operator registry whose adapters call
 * yvex_backend_command and yvex_rocm_info_command with the adapter argv (src/cli/main.c
 * routes "backend" and "cuda-info" the same way); this program is that routing and nothing
 * else.  Exit codes: 0 success, 2 grammar, 5 backend unsupported on this machine.
 */
#include <stdio.h>
#include <string.h>

#include "yvex_rocm.h"
#include "yvex_rocm_operations.h"

static int usage(FILE *fp, int code)
{
    fprintf(fp, "usage: yvex-rocm inspect backend rocm\n"
                "       yvex-rocm inspect rocm [bandwidth]\n");
    return code;
}

int main(int argc, char **argv)
{
    char *adapter[4];
    int count = 0, index;
    if (argc == 2 && (strcmp(argv[1], "--help") == 0 || strcmp(argv[1], "-h") == 0))
        return usage(stdout, 0);
    if (argc < 3 || argc > 5 || strcmp(argv[1], "inspect") != 0) return usage(stderr, 2);
    adapter[count++] = argv[0];
    if (strcmp(argv[2], "backend") == 0) {
        adapter[count++] = "backend";
        for (index = 3; index < argc; ++index) adapter[count++] = argv[index];
        return yvex_backend_command(count, adapter);
    }
    if (strcmp(argv[2], "rocm") == 0) {
        adapter[count++] = "rocm-info";
        for (index = 3; index < argc; ++index) adapter[count++] = argv[index];
        return yvex_rocm_info_command(count, adapter);
    }
    return usage(stderr, 2);
}
