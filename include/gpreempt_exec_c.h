/*
 * gpreempt_exec_c.h — C view of the C++ executor classes (include/executor.h, include/model.h)
 * for callers that bind through an FFI (ctypes, cgo, JNI) instead of linking C++.
 * Every function forwards to the method of foo::Executor / foo::BLPExecutor named in its
 * comment, which in turn replaces the method of the same name in the reference
 * (include/executor.h:14-84).  Results are the `Status` values of include/util/common.h
 * (0 = Succ) unless stated otherwise.
 */
#ifndef GPREEMPT_EXEC_C_H
#define GPREEMPT_EXEC_C_H
#include <stddef.h>
#include "gpreempt_hip.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef void *gpx_executor;

gpx_executor gpx_create(int block_level_preemptible); /* 0: foo::BaseExecutor, 1: foo::BLPExecutor */
void gpx_destroy(gpx_executor e);
int gpx_init(gpx_executor e, const char *workload);                 /* Executor::init */
int gpx_set_input(gpx_executor e, const char *key, void *value, size_t len, gp_stream s);  /* Executor::set_input */
int gpx_get_output(gpx_executor e, const char *key, void *value, size_t len, gp_stream s); /* Executor::get_output */
size_t gpx_get_data_size(gpx_executor e, const char *key);          /* Executor::get_data_size */
int gpx_execute(gpx_executor e, gp_stream s);                        /* Executor::execute */
int gpx_launch_kernel(gpx_executor e, size_t idx, gp_stream s);      /* Executor::launch_kernel */
size_t gpx_get_kernel_num(gpx_executor e);                           /* Executor::get_kernel_num */
int gpx_capture_graph(gpx_executor e, gp_stream s);                  /* Executor::capture_graph; 0 when a graph is in use afterwards */
int gpx_uses_program(gpx_executor e);                                /* 1 when capture_graph built the persistent program */
void gpx_clear(gpx_executor e);                                      /* Executor::clear */

/* BLPExecutor only (Status::Fail on a BaseExecutor) */
int gpx_set_flag(gpx_executor e, void *dp_stop);                     /* BLPExecutor::dpStop = dp_stop */
int gpx_set_running(gpx_executor e, int running);                    /* BLPExecutor::running = running */
int gpx_resume(gpx_executor e, gp_stream s);                         /* BLPExecutor::resume */
int gpx_get_stop_point(gpx_executor e, gp_stream s, int *stop_index);/* BLPExecutor::getStopPoint */
int gpx_last_stop_index(gpx_executor e);                             /* value read by the last getStopPoint / resume */
int gpx_inject_preempt(gpx_executor e, int kernel, int claim);       /* BLPExecutor::inject_preempt (test hook) */
int gpx_read_counters(gpx_executor e, int *out, size_t n);           /* BLPExecutor::read_counters */
int gpx_reset_counters(gpx_executor e, gp_stream s);                 /* BLPExecutor::reset_counters */

/* Model introspection (foo::Model::get_storage_info / get_kernel_info) */
size_t gpx_storage_num(gpx_executor e);
/* dims = {kind, o, i, r, s, c, h, w}: kind 0 plain, 1 conv weight stored OIHW on disk, 2 dense over a CHW flatten */
int gpx_storage_info(gpx_executor e, size_t idx, char *name, size_t name_len, char *stype, size_t stype_len,
                     size_t *bytes, int *is_param, size_t *disk_elems, int dims[8]);
int gpx_kernel_info(gpx_executor e, size_t idx, char *name, size_t name_len, double *flops, double *bytes,
                    int *total_blocks, int *grid);
int gpx_read_storage(gpx_executor e, const char *key, void *out, size_t len); /* blocking Model::get */

/* Graph workloads ("cc", "bfs", "pagerank", "sssp"; GraphCompute classes of the reference's
 * include/workloads/graphcompute.h).  info = {vertices, edges, iterations of the last execute,
 * preemptions so far, kernels launched so far}; result keys: "comp" (u64 per vertex), "label" (u32),
 * "value" (f32), "cost" (u32).  gpx_set_lc_tasks sets the count of active latency-critical tasks
 * that the executor's loop waits on when it has been stopped (BLPExecutor::set_lc_be_tasks is
 * called with counters the handle owns). */
int gpx_graph_info(gpx_executor e, unsigned long long info[5]);
size_t gpx_graph_result_bytes(gpx_executor e, const char *key);
int gpx_graph_result(gpx_executor e, const char *key, void *out, size_t len);
int gpx_graph_inject_preempt(gpx_executor e, int iteration, int kernel, int claim); /* BLPExecutor::inject_preempt_graph */
int gpx_set_lc_tasks(gpx_executor e, int n);
int gpx_set_graph_path(gpx_executor e, const char *base);           /* Executor::set_graph_path (before gpx_init) */
/* Writes a seeded random graph as <base>.col / .dst / .val in the reference's file format. */
int gpx_write_synthetic_graph(const char *base, unsigned long long vertices, unsigned degree, unsigned long long seed);

/* "miniweather" workload only: domain mass and total energy of the current state
 * (SciComputeBlp::reductions, reference src/workloads/miniweather.tr.cu:906-932); blocking. */
int gpx_miniweather_reductions(gpx_executor e, double *mass, double *te);

/* Multi-tenant scenario runner: the role of the reference's client executables
 * (src/cuda-clients/blpclient.cpp main() and the programs under src/common-clients) over a DISB task file
 * (config/A.json schema) with an extra "policy" key: "wb" (block-level preemption, HP waits for
 * the drain as blpclient.cpp:189 does), "wb-async" (HP submits at once), "np" (no preemption,
 * baseclient.cpp), "seq" (seqclient.cpp), "lco" (high-priority tasks only, rtonlyclient.cpp).
 * The JSON report is written to `report` (NUL-terminated, truncated to report_len). */
int gpx_run_scenario(const char *config_json, char *report, size_t report_len);
/* Per-kernel preemption / resume latency of one best-effort model (BASELINE config 2): `trials` inferences, each
 * stopped at a random instant by the host and resumed (the protocol of src/tests/test-dnn-blp.cpp:36-42).
 * use_graph: 0 = BLPExecutor::execute launches every kernel at once, 1 = the captured form (whole-model program),
 * 2 = kernel by kernel with a bounded queue, as the scenario runner feeds a best-effort tenant. */
int gpx_preempt_probe(const char *workload, int trials, int use_graph, unsigned long long seed, char *report, size_t report_len);
/* Parses a TVM_MODEL_PARAMS file (ModelParamParser::parse_from_file, reference src/model.cpp:15-55):
 * returns the number of tensors (-1: missing or malformed); when `key` names a tensor, up to n of
 * its values are copied to `out` and *len receives its length. */
long gpx_parse_params(const char *path, const char *key, float *out, size_t n, size_t *len);

/* Reads an exported model directory's mod.json + host.json as Model::load_from_json of the
 * reference does (src/model.cpp:128-235) and, when ops_json is given, the operator-attribute
 * sidecar (include/tvm_export.h), checked against the export.  The JSON report holds "storages"
 * (name, stype, size), "kernels" (name, func, launch_params, args_index), "global_len",
 * "heads_index", "ops" and "error".  Needs no GPU. */
int gpx_parse_tvm_export(const char *device_json, const char *host_json, const char *ops_json, char *report, size_t report_len);
/* The native kernel list that an export plus its sidecar maps to (foo::build_export_graph, include/tvm_export.h),
 * in element type `dtype` ("f32" "f16" "bf16"; NULL or "" = the export's own): what Model::load_model runs when
 * the model directory holds an ops.json, where the reference loads the export's own device code
 * (src/model.cpp:84-98).  The JSON report holds "storages" (name, stype, size, is_param, kind, disk_elems),
 * "kernels" (name, args = storage names, params) and "error".  Needs no GPU. */
int gpx_plan_tvm_export(const char *device_json, const char *host_json, const char *ops_json, const char *dtype, char *report, size_t report_len);

/* include/gpreempt.h through the C view.  gpx_set_priority = NvRmQuery + set_priority on the
 * tenant's stream (reference src/cuda-clients/gpreemptclient.cpp:170-177); 0 or -1 as the reference.
 * A domain is a foo::PreemptDomain (one flag word per priority boundary); its handle is what
 * hipGetFd() returns and hipSuspendStreams / hipResumeStreams take (reference
 * include/gpreempt.h:191-194), with priority levels in the place of hardware queue ids.
 * gpx_domain_flag returns the device-visible address of the word that level `priority` (>= 1)
 * obeys: the value for BLPExecutor::dpStop (gpx_set_flag).  gpx_domain_begin / _end announce and
 * retire a request of `priority`, which raises / lowers the words of every lower level. */
int gpx_set_priority(gp_stream s, int priority);
int gpx_domain_create(int levels);   /* handle >= 0, or -1 */
int gpx_domain_destroy(int fd);
int gpx_get_fd(void);                /* hipGetFd(): the newest live domain, -1 when there is none */
void *gpx_domain_flag(int fd, int priority);
int gpx_domain_flag_value(int fd, int priority);  /* the word's current value on the host side; -1: no such word */
int gpx_domain_begin(int fd, int priority);
int gpx_domain_end(int fd, int priority);
int gpx_suspend_streams(int fd, const int *levels, int n);  /* hipSuspendStreams */
int gpx_resume_streams(int fd, const int *levels, int n);   /* hipResumeStreams */

#ifdef __cplusplus
}
#endif
#endif
