/* The public header compiles as C99 and the library links from a plain C program: every call below is refused by
 * argument validation (or is a size query), so no GPU is needed.  Built and run by tests/test_abi.py. */
#include <stdio.h>
#include <stddef.h>
#include "egs_hip.h"

#define EXPECT(cond) do { if (!(cond)) { printf("FAILED: %s (line %d)\n", #cond, __LINE__); return 1; } } while (0)

int main(void)
{
    egs_dims d = {64, 256, 32, 32, 128, 64};
    void *p = (void *)(size_t)0x1000;
    unsigned long long id = 7;
    EXPECT(egs_abi_version() >= 1);
    EXPECT(egs_status_string(0) != NULL && egs_status_string(EGS_ERR_WORKSPACE) != NULL);
    EXPECT(egs_workspace_bytes(EGS_OP_GEMM_SCATTER, EGS_SCATTER_DETERMINISTIC, &d, EGS_BF16) == 0);
    EXPECT(egs_routing_table_bytes(&d, EGS_BF16) > 0);
    EXPECT(egs_expert_mlp_supported(&d, EGS_BF16) == 1);
    EXPECT(egs_gather_gemm(NULL, p, p, p, NULL, &d, 256 * 128, 128, EGS_BF16, EGS_BF16, EGS_IND_I64, EGS_W_EIJ, NULL) == EGS_ERR_NULL_POINTER);
    EXPECT(egs_expert_gather_forward(p, p, p, p, &d, 256 * 128, 128, 99, EGS_IND_I64, NULL) == EGS_ERR_BAD_DTYPE);
    EXPECT(egs_expert_scatter_forward(p, p, p, p, NULL, 0, &d, EGS_BF16, EGS_IND_I64, 9, NULL) == EGS_ERR_BAD_MODE);
    EXPECT(egs_expert_gather_forward_table(p, p, p, p, p, 16, &d, 256 * 128, 128, EGS_BF16, EGS_IND_I64, NULL) == EGS_ERR_ALIGNMENT
           || egs_expert_gather_forward_table(p, p, p, p, p, 16, &d, 256 * 128, 128, EGS_BF16, EGS_IND_I64, NULL) == EGS_ERR_WORKSPACE);
    EXPECT(egs_stream_capture_id(NULL, NULL) == EGS_ERR_NULL_POINTER);
    (void)id;
    printf("ok %d\n", egs_abi_version());
    return 0;
}
