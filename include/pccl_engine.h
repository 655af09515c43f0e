/*
 * pccl_engine.h -- C ABI of the host layer, libpccl_engine.so: the engine
 * (register a compiled collective by name, run it), the type registry and the
 * schedule generators.  This is what a binding for another language wraps; the
 * C++ classes behind it keep the reference's names (engine_c::Engine,
 * TypeRegistry, DeviceBase ...).
 *
 * Every function returns 0 or a negative code; C++ exceptions are caught at
 * this boundary and their text is kept for pccl_engine_last_error().
 */
#ifndef PCCL_ENGINE_H
#define PCCL_ENGINE_H

#ifdef __cplusplus
extern "C" {
#endif

#define PCCL_ENGINE_OK 0
#define PCCL_ENGINE_ERR (-1)          /* an exception was caught; see last_error */
#define PCCL_ENGINE_ERR_ARG (-2)      /* null handle / pointer */

/* ---- Engine: include/engine.h:13-23, csrc/python_api.cc:13-20 --------------- */
int pccl_engine_create(int rank, int world_size, void **engine);  /* Engine(int, int), engine.h:15 */
int pccl_engine_destroy(void *engine);
int pccl_engine_init(void *engine);                                /* initEngine(), engine.cc:42-100 */
/* regOp(name, filepath), engine.h:18: filepath holds a schedule in the text format of
 * pccl_amd/csrc/host/schedule.h */
int pccl_engine_reg_op(void *engine, const char *name, const char *filepath);
/* regOp from memory: `text` is the contents such a file would have */
int pccl_engine_reg_op_text(void *engine, const char *name, const char *text);
/* exeOp(name, input, output), engine.h:19: device addresses and byte sizes of the two
 * tensors; asynchronous on `stream` (a hipStream_t, NULL = default stream) */
int pccl_engine_exe_op(void *engine, const char *name, const void *input, long input_bytes, void *output,
                       long output_bytes, void *stream);
/* waits for `stream` and verifies *completed_operator == *total_operator (operator.h:32-33) */
int pccl_engine_wait_op(void *engine, const char *name, void *stream);
/* (workspace, signals) of a device type, BufferManager::getDevBuffer, chunk.h:46 */
int pccl_engine_get_dev_buffer(void *engine, const char *device_name, void **workspace, void **signals,
                               long *workspace_bytes);
/* number of operators / devices / elements per device of a registered op */
int pccl_engine_op_info(void *engine, const char *name, int *n_ops, int *devices, long *elems_per_device,
                        int *elem_bytes);
/* exportEndpoint / joinCluster / exitCluster (engine.h:21-23): cluster control plane, absent
 * from this build; these return PCCL_ENGINE_ERR with an explanatory text */
int pccl_engine_export_endpoint(void *engine, char *buf, int buf_len);
int pccl_engine_join_cluster(void *engine, const char *master_endpoint);
int pccl_engine_exit_cluster(void *engine);

/* ---- one reduce-copy through the plugin layer (HipExecutor::reduceCopy) -------------- */
/* dtype / compute are TypeRegistry NAMES ("bf16", "sum", ...) */
int pccl_engine_reduce_copy(const char *dtype, const char *compute, const void *const *ins, int n_in,
                            void *const *outs, int n_out, long count, void *stream);

/* ---- TypeRegistry: include/base/registry.h:25-43 ------------------------------------- */
int pccl_registry_type_id(const char *name, int *id);            /* getTypeId  */
int pccl_registry_type_name(int id, char *buf, int buf_len);     /* getTypeName */
/* kind: 0 primitive, 1 data, 2 compute, 3 device, 4 executor */
int pccl_registry_register(int kind, const char *name, int *id); /* register*Type */
int pccl_registry_register_compat(const char *executor, const char *type_name);
int pccl_registry_is_compatible(const char *executor, const char *type_name, int *yes);
/* device type names, '\n'-separated (getDeviceTypes) */
int pccl_registry_device_types(char *buf, int buf_len);

/* ---- DeviceBase plugins: include/base/device.h:8-43 ---------------------------------- */
int pccl_device_allocator_available(const char *device_name, int *yes);
int pccl_device_allocate(const char *device_name, long nbytes, void **p);  /* *p == NULL on failure */
int pccl_device_deallocate(const char *device_name, void *p);
int pccl_device_ipc_available(const char *device_name, int *yes);

/* ---- launch options: include/common/environ.h:11-37, python_api.cc:24-27 ------------- */
int pccl_env_list_opt(char *buf, int buf_len);                   /* '\n'-separated */
int pccl_env_get(const char *name, char *buf, int buf_len);
int pccl_env_register_opt(const char *name);                     /* registerOpt */

/* ---- schedule generators (native side of pccl/lang) ---------------------------------- */
/* Each writes a schedule file that pccl_engine_reg_op loads. */
int pccl_schedule_write_ring_allreduce(const char *path, const char *dtype, const char *compute, int devices,
                                       long chunk_elems);
int pccl_schedule_write_direct_allreduce(const char *path, const char *dtype, const char *compute, int devices,
                                         long slice_elems);
/* kind: "ring_allreduce", "direct_allreduce", "ring_reduce_scatter", "ring_all_gather", "all_to_all"
 * (elems = per chunk / slice) or "broadcast" (elems in all, from device `root`; root is ignored otherwise). */
int pccl_schedule_write_collective(const char *path, const char *kind, const char *dtype, const char *compute,
                                   int devices, long elems, int root);
int pccl_schedule_write_small_message(const char *path, const char *dtype, int devices, int n_slices, int n_extra,
                                      unsigned long seed, long lo_bytes, long hi_bytes);
/* Parses and validates `path`; reports its shape and, if order != NULL, the op ids in the
 * order pccl/lang/utils/graph.py:94-112 would execute them (order_len >= n_ops). */
int pccl_schedule_inspect(const char *path, int *n_ops, int *devices, long *elems_per_device, int *order,
                          int order_len);

const char *pccl_engine_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
