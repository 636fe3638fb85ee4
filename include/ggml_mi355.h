/*
 * Entry points of libggml-mi355.so, the ggml backend plug-in for one AMD Instinct MI355X.
 *
 * These are exactly the two symbols llama.cpp's backend registry resolves with dlsym() when
 * it loads a backend library (ggml/src/ggml-backend-reg.cpp:229-245; typedefs
 * ggml_backend_init_t / ggml_backend_score_t in ggml/src/ggml-backend-impl.h:208-214, the
 * macros that normally generate them at :215-251).  Everything else the host uses is reached
 * through the function-pointer tables of the returned registration object
 * (struct ggml_backend_reg / _device / _buffer_type / _buffer / ggml_backend,
 * ggml/src/ggml-backend-impl.h:17-207), which the plug-in fills:
 *
 *   reg         get_name "MI355X", get_device_count, get_device, get_proc_address (none)
 *   device      GPU type; get_memory (hipMemGetInfo); init_backend; get_buffer_type; a pinned host
 *               buffer type (hipHostMalloc) for the tensors the CPU backend hands over;
 *               supports_op / supports_buft; event_new / event_free / event_synchronize (HIP events
 *               without timing); caps: async, host_buffer and events true, buffer_from_host_ptr false
 *   buffer type hipMalloc-backed, alignment 256, alloc size = ggml_nbytes
 *   buffer      set/get/memset/cpy_tensor and clear; set/get apply / undo the 16-byte-aligned
 *               device row layout for Q4_0, Q8_0 and Q6_K tensors
 *   backend     one HIP stream; set/get_tensor_async, cpy_tensor_async (host tensors of the CPU backend
 *               and tensors of this backend) and event_record / event_wait on it; graph_compute walks the graph once,
 *               matching runs of nodes (norm -> weight -> products -> rope -> cache store, gate/up
 *               -> SiLU*up -> down, ...) to one fused kernel each, records the launches of a
 *               decode-shaped graph into a HIP graph keyed by the graph's signature and replays
 *               it on later calls; synchronize waits for the stream
 *
 * The library has no link-time dependency on libggml-base: the handful of ggml symbols it calls
 * (ggml_backend_buffer_init, ggml_nbytes, ggml_is_contiguous, ...) resolve against the host
 * process that loads it.
 */
#ifndef GGML_MI355_H
#define GGML_MI355_H

#ifdef __cplusplus
extern "C" {
#endif

struct ggml_backend_reg;

/* Registration object of the backend (api_version = GGML_BACKEND_API_VERSION, 1).  Static for
 * the life of the process.  Replaces e.g. ggml_backend_cuda_reg (ggml/src/ggml-cuda/ggml-cuda.cu:3394). */
struct ggml_backend_reg *ggml_backend_init(void);

/* 0 when no gfx950 device is visible (the registry then skips the library), 100 otherwise. */
int ggml_backend_score(void);

#ifdef __cplusplus
}
#endif
#endif /* GGML_MI355_H */
