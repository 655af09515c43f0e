#include "plugin_common.h"
using pccl_host::fail;
extern "C" {
int pccl_hip_graph_create(const pccl_op_desc *, int, long, void **) { return fail(PCCL_ERR_UNSUPPORTED, "graph path not built yet"); }
int pccl_hip_graph_run(void *, void *) { return fail(PCCL_ERR_UNSUPPORTED, "graph path not built yet"); }
int pccl_hip_graph_status(void *, void *, unsigned int *, unsigned int *) { return fail(PCCL_ERR_UNSUPPORTED, "graph path not built yet"); }
int pccl_hip_graph_rebind(void *, const void *, const void *, long, void *) { return fail(PCCL_ERR_UNSUPPORTED, "graph path not built yet"); }
int pccl_hip_graph_info(void *, void **, int *, int *) { return fail(PCCL_ERR_UNSUPPORTED, "graph path not built yet"); }
int pccl_hip_graph_destroy(void *) { return PCCL_OK; }
}
