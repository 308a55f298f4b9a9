/* Internal declarations of the HIP layer (plain C types only).  The public
 * subset is repeated in include/alphasparse_amd.h. */
#pragma once
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
const char *as_hip_last_error(void);
int as_hip_device_count(void);
int as_hip_init(int device);
int as_hip_static_scratch(int device, void **ptr, uint64_t *bytes);
int as_hip_device_info(int device, char *name, int name_cap, int *cu_count, int *wave_size, uint64_t *lds_per_block,
                       uint64_t *global_mem);
int as_hip_compile(const char *src, const char *arch, const char *const *opts, int n_opts, void **code,
                   uint64_t *code_size, char **log);
void as_hip_free_host(void *p);
int as_hip_module_load(const void *code, void **module);
int as_hip_module_unload(void *module);
int as_hip_get_kernel(void *module, const char *name, void **fn);
int as_hip_alloc(void **p, uint64_t bytes);
int as_hip_free(void *p);
int as_hip_h2d(void *dst, const void *src, uint64_t bytes);
int as_hip_d2h(void *dst, const void *src, uint64_t bytes);
int as_hip_memset_async(void *dst, int value, uint64_t bytes, void *stream);
int as_hip_stream_create(void **stream);
int as_hip_stream_destroy(void *stream);
int as_hip_stream_sync(void *stream);
int as_hip_device_sync(void);
int as_hip_event_create(void **ev);
int as_hip_event_destroy(void *ev);
int as_hip_event_record(void *ev, void *stream);
int as_hip_event_sync(void *ev);
int as_hip_event_elapsed_ms(void *start, void *stop, float *ms);
int as_hip_stream_wait_event(void *stream, void *ev);
int as_hip_graph_capture_begin(void *stream);
int as_hip_graph_capture_end(void *stream, void **graph_exec);
int as_hip_graph_launch(void *graph_exec, void *stream);
int as_hip_graph_destroy(void *graph_exec);
int as_hip_mem_info(uint64_t *free_bytes, uint64_t *total_bytes);
int as_hip_launch(void *fn, unsigned grid, unsigned block, unsigned lds_bytes, void *stream, void **args);
#ifdef __cplusplus
}
#endif
