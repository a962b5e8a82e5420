/* A plain C99 client of include/nanoep_hip.h: proves that the header is C (no C++, HIP or torch
 * types) and that a caller can link the shared library directly.  It calls only entry points
 * that need no GPU and prints what tests/test_cabi_library.py checks. */
#include <stdio.h>

#include "nanoep_hip.h"

int main(void) {
    int64_t window[5] = {0, 0, 0, 0, 0};
    const int status = nanoep_window_layout(2, 8, 256, 2, 4, 0, window);
    printf("abi %d status %d window %lld %lld %lld %lld %lld\n", nanoep_abi_version(), status, (long long)window[0],
           (long long)window[1], (long long)window[2], (long long)window[3], (long long)window[4]);
    printf("invalid %d '%s'\n", nanoep_dispatch(NULL, NULL, NULL, NULL, NULL, NULL, 0, NULL, NULL, 0, 0, 0, 7, 2, 4, 1, 0, 0, NULL, NULL, NULL, 0, NULL),
           nanoep_status_string(NANOEP_ERR_INVALID_ARGUMENT));
    printf("sizes %lld %d %lu\n", (long long)nanoep_slot_order_entries(4096, 8, 256), nanoep_layout_block_tokens(4096, 256, 7168),
           (unsigned long)(nanoep_layout_workspace_bytes(4096, 8, 256) > 0));
    return 0;
}
