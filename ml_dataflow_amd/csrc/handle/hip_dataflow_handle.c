/*
 * hip_dataflow_handle.c -- Dataflow_Handle for one AMD GPU, written against the HIP runtime C API.
 *
 * Fills every function pointer of the handle declared in include/dataflow_amd.h.  Plays the role of
 * backends/nvidia/src/handle/src/cuda_dataflow_handle.c (init :865-1105, registration :151-348,
 * submit_op :354-448, dependencies :470-560, memory/transfers :565-760) for COMPUTE_HSA.
 *
 * Design points that differ from the CUDA backend:
 *   - no driver-API context juggling: a HIP device has one primary context, the handle just makes its
 *     device current before every call that needs it;
 *   - every stream is created at the default priority (requested priorities are recorded, not applied);
 *   - native code is a gfx950 code object (.hsaco) loaded with hipModuleLoad; kernels are launched with
 *     hipModuleLaunchKernel and receive op->op_args unchanged as their parameter list;
 *   - set_mem on a stream is a hipMemsetD8Async; callers that capture graphs must not route set_mem
 *     into a capture.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include "dataflow_amd.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <dlfcn.h>

#define HIP_OK(call, what, fail_stmt) do { \
	hipError_t _e = (call); \
	if (_e != hipSuccess) { \
		fprintf(stderr, "Error: %s failed: %s (%d)...\n", what, hipGetErrorString(_e), (int) _e); \
		fail_stmt; \
	} } while (0)

static int make_current(Dataflow_Handle * h) {
	HIP_OK(hipSetDevice(h->device_id), "hipSetDevice", return -1);
	return 0;
}

static hipStream_t * handle_streams(Dataflow_Handle * h) { return (hipStream_t *) h->streams; }
static hipEvent_t * handle_events(Dataflow_Handle * h) { return (hipEvent_t *) h->stream_states; }

/* stream_id -1 is the null stream (cuda_dataflow_handle.c:364-373) */
static int resolve_stream(Dataflow_Handle * h, int stream_id, hipStream_t * out, const char * what) {
	if (stream_id == -1) {
		*out = NULL;
		return 0;
	}
	if (stream_id < 0 || stream_id >= h->num_streams) {
		fprintf(stderr, "Error: cannot %s on stream id %d, when device only has %d streams. Null stream specified by -1...\n", what, stream_id, h->num_streams);
		return -1;
	}
	*out = handle_streams(h)[stream_id];
	return 0;
}

/* ------------------------------------------------------------------ op table hash */

/* last 8 fingerprint bytes, big-endian, modulo the table size (cuda_dataflow_handle.c:31-44) */
static uint64_t hip_op_table_hash_func(void * op_fingerprint, uint64_t table_size) {
	const uint8_t * tail = (const uint8_t *) op_fingerprint + DATAFLOW_OP_IDENTIFIER_FINGERPRINT_NUM_BYTES - 8;
	uint64_t v = 0;
	for (int i = 0; i < 8; i++) {
		v = (v << 8) | (uint64_t) tail[i];
	}
	return v % table_size;
}

/* ------------------------------------------------------------------ profiler (roctx, resolved lazily) */

typedef int (*roctx_push_fn)(const char *);
typedef int (*roctx_pop_fn)(void);
typedef int (*roctx_name_thread_fn)(const char *);
typedef int (*roctx_name_device_fn)(const char *, int);
typedef int (*roctx_name_stream_fn)(const char *, const void *);
static roctx_push_fn roctx_push = NULL;
static roctx_pop_fn roctx_pop = NULL;
static roctx_name_thread_fn roctx_name_thread = NULL;      /* the naming calls exist in the rocprofiler-sdk marker library only */
static roctx_name_device_fn roctx_name_device = NULL;
static roctx_name_stream_fn roctx_name_stream = NULL;
static int roctx_tried = 0;

static void roctx_resolve(void) {
	if (roctx_tried) {
		return;
	}
	roctx_tried = 1;
	const char * names[] = {"librocprofiler-sdk-roctx.so", "libroctx64.so"};
	for (int i = 0; i < 2 && !roctx_push; i++) {
		void * lib = dlopen(names[i], RTLD_LAZY | RTLD_LOCAL);
		if (lib) {
			roctx_push = (roctx_push_fn) dlsym(lib, "roctxRangePushA");
			roctx_pop = (roctx_pop_fn) dlsym(lib, "roctxRangePop");
			if (!roctx_push || !roctx_pop) {
				roctx_push = NULL;
				roctx_pop = NULL;
				continue;
			}
			roctx_name_thread = (roctx_name_thread_fn) dlsym(lib, "roctxNameOsThread");
			roctx_name_device = (roctx_name_device_fn) dlsym(lib, "roctxNameHipDevice");
			roctx_name_stream = (roctx_name_stream_fn) dlsym(lib, "roctxNameHipStream");
		}
	}
}

static int hip_profiler_start(void) { return (hipProfilerStart() == hipSuccess) ? 0 : -1; }
static int hip_profiler_stop(void) { return (hipProfilerStop() == hipSuccess) ? 0 : -1; }
/* The reference forwards these to NVTX (nvtxNameCuDeviceA, nvtxNameCuContextA, nvtxNameCuStreamA, nvtxNameOsThreadA:
 * backends/nvidia/src/handle/src/cuda_profiler.c:49-70); here they go to the marker library's naming calls where it has
 * them (a profiler that listens labels the device, the stream or the calling thread) and do nothing otherwise.  HIP has
 * no context object to name: the handle's name labels its device. */
static void hip_profiler_name_device(Dataflow_Handle * h, const char * name) {
	roctx_resolve();
	if (h && name && roctx_name_device) {
		(void) roctx_name_device(name, h->device_id);
	}
}
static void hip_profiler_name_handle(Dataflow_Handle * h, const char * name) {
	hip_profiler_name_device(h, name);
}
static void hip_profiler_name_stream(Dataflow_Handle * h, int stream_id, const char * name) {
	if (stream_id < 0 || stream_id >= h->num_streams) {
		fprintf(stderr, "Error: cannot name stream with id %d, when device only has %d streams...\n", stream_id, h->num_streams);
		return;
	}
	roctx_resolve();
	if (name && roctx_name_stream) {
		(void) roctx_name_stream(name, (const void *) handle_streams(h)[stream_id]);
	}
}
static void hip_profiler_name_thread(Dataflow_Handle * h, const char * name) {
	(void) h;
	roctx_resolve();
	if (name && roctx_name_thread) {
		(void) roctx_name_thread(name);
	}
}
static int hip_profiler_range_push(const char * message) {
	roctx_resolve();
	return roctx_push ? roctx_push(message) : 0;
}
static int hip_profiler_range_pop(void) {
	roctx_resolve();
	return roctx_pop ? roctx_pop() : 0;
}

/* ------------------------------------------------------------------ ops */

static int hip_get_num_procs(Dataflow_Handle * h) {
	return ((Hip_Device_Info *) h->device_info)->cu_count;
}

static int hip_register_native_code(Dataflow_Handle * h, char * native_code_filename, char * native_code_config_lib_filename,
									int num_funcs, Op_Skeleton * func_op_skeletons, char ** func_symbols,
									char ** func_set_launch_symbols, char ** func_init_symbols) {
	if (h->num_native_function_libs >= MAX_NATIVE_FUNCTION_LIBS) {
		fprintf(stderr, "Error: cannot register more than %d native function libs...\n", MAX_NATIVE_FUNCTION_LIBS);
		return -1;
	}
	if (make_current(h)) {
		return -1;
	}
	hipModule_t module;
	HIP_OK(hipModuleLoad(&module, native_code_filename), "hipModuleLoad", {
		fprintf(stderr, "Error: unable to load function lib from path: %s...\n", native_code_filename);
		return -1; });

	void * config_lib = dlopen(native_code_config_lib_filename, RTLD_NOW | RTLD_LOCAL);
	if (!config_lib) {
		fprintf(stderr, "Error: could not load function config shared lib with dlopen() from path: %s (%s)\n", native_code_config_lib_filename, dlerror());
		hipModuleUnload(module);
		return -1;
	}

	int added = 0;
	for (int i = 0; i < num_funcs; i++) {
		const char * sym = func_symbols[i];
		if (!sym) {
			continue;
		}
		if (!func_set_launch_symbols || !func_set_launch_symbols[i]) {
			fprintf(stderr, "Error: set launch symbol not set for native function %s, but is required for native functions...\n", sym);
			continue;
		}
		Hip_Function fn;
		memset(&fn, 0, sizeof(fn));
		fn.is_native = true;
		hipFunction_t f;
		if (hipModuleGetFunction(&f, module, sym) != hipSuccess) {
			fprintf(stderr, "Error: failed to load function #%d with name %s from function lib...\n", i, sym);
			continue;
		}
		fn.function_handle = (void *) f;
		fn.function_config.func_max_threads_per_block = ((Hip_Device_Info *) h->device_info)->max_threads_per_block;
		fn.function_config.func_max_lds = ((Hip_Device_Info *) h->device_info)->max_lds_per_block;
		if (func_init_symbols && func_init_symbols[i]) {
			Hip_Set_Func_Attribute set_attr = (Hip_Set_Func_Attribute) dlsym(config_lib, func_init_symbols[i]);
			if (!set_attr) {
				fprintf(stderr, "Error: failed to load symbol to initialize function #%d with name %s and attribute setting function as %s...\n", i, sym, func_init_symbols[i]);
				continue;
			}
			if (set_attr(h, &fn)) {
				fprintf(stderr, "Error: failed to set function attributes for function #%d with name %s...\n", i, sym);
				continue;
			}
		}
		fn.set_launch_config = (int (*)(Hip_Launch_Config *, Dataflow_Handle *, Hip_Function *, Op *)) dlsym(config_lib, func_set_launch_symbols[i]);
		if (!fn.set_launch_config) {
			fprintf(stderr, "Error: failed to get function pointer to launch config for function #%d with name %s and set_launch_config function name as %s\n", i, sym, func_set_launch_symbols[i]);
			continue;
		}
		memcpy(&fn.op_skeleton, &func_op_skeletons[i], sizeof(Op_Skeleton));
		if (dataflow_insert_table(&h->op_table, fn.op_skeleton.identifier.fingerprint, &fn)) {
			fprintf(stderr, "Error: failed to insert op for function #%d with name %s to op table...\n", i, sym);
			continue;
		}
		added++;
	}
	if (added == 0) {
		fprintf(stderr, "Error: no functions were added to op table...\n");
		hipModuleUnload(module);
		return -1;
	}
	h->native_function_libs[h->num_native_function_libs++] = (void *) module;
	h->num_ops += added;
	return added;
}

static int hip_register_external_code(Dataflow_Handle * h, char * external_code_filename, int num_funcs,
									  Op_Skeleton * func_op_skeletons, char ** func_symbols, char ** func_init_symbols) {
	if (make_current(h)) {
		return -1;
	}
	void * lib = dlopen(external_code_filename, RTLD_NOW | RTLD_LOCAL);
	if (!lib) {
		fprintf(stderr, "Error: could not open external library with path: %s (%s)\n", external_code_filename, dlerror());
		return -1;
	}
	int added = 0;
	for (int i = 0; i < num_funcs; i++) {
		const char * sym = func_symbols[i];
		if (!sym) {
			continue;
		}
		Hip_Function fn;
		memset(&fn, 0, sizeof(fn));
		fn.is_native = false;
		fn.hip_external_func = (External_Lib_Func) dlsym(lib, sym);
		if (!fn.hip_external_func) {
			fprintf(stderr, "Error: could not obtain function symbol %s from external lib %s...\n", sym, external_code_filename);
			continue;
		}
		if (func_init_symbols && func_init_symbols[i]) {
			External_Lib_Func_Init init = (External_Lib_Func_Init) dlsym(lib, func_init_symbols[i]);
			if (!init) {
				fprintf(stderr, "Error: could not get ref to initialization function %s, for external function %s\n", func_init_symbols[i], sym);
				continue;
			}
			if (init(h, (void *) &fn)) {
				fprintf(stderr, "Error: initialization function %s, for external function %s returned an error...\n", func_init_symbols[i], sym);
				continue;
			}
		}
		memcpy(&fn.op_skeleton, &func_op_skeletons[i], sizeof(Op_Skeleton));
		if (dataflow_insert_table(&h->op_table, fn.op_skeleton.identifier.fingerprint, &fn)) {
			fprintf(stderr, "Error: failed to insert op for function #%d with name %s to op table...\n", i, sym);
			continue;
		}
		added++;
	}
	h->num_ops += added;
	return added;
}

static int hip_submit_op(Dataflow_Handle * h, Op * op, int stream_id) {
	hipStream_t stream;
	if (resolve_stream(h, stream_id, &stream, "submit op")) {
		fprintf(stderr, "Error: op had nickname %s...\n", op->op_skeleton.header.op_nickname);
		return -1;
	}
	Hip_Function * fn = NULL;
	long at = dataflow_find_table(&h->op_table, op->op_skeleton.identifier.fingerprint, false, (void **) &fn);
	if (at < 0 || !fn) {
		fprintf(stderr, "Error: failed to find op with nickname %s and matching dtypes...\n", op->op_skeleton.header.op_nickname);
		return -1;
	}
	if (make_current(h)) {
		return -1;
	}
	if (fn->is_native) {
		Hip_Launch_Config cfg;
		memset(&cfg, 0, sizeof(cfg));
		if ((fn->set_launch_config)(&cfg, h, fn, op)) {
			fprintf(stderr, "Error: failed to correctly set launch config for op with nickname %s...\n", op->op_skeleton.header.op_nickname);
			return -1;
		}
		/* a launch config with an empty grid means "nothing to do" (e.g. zero rows) */
		if (cfg.gridDimX == 0 || cfg.gridDimY == 0 || cfg.gridDimZ == 0) {
			return 0;
		}
		HIP_OK(hipModuleLaunchKernel((hipFunction_t) fn->function_handle, cfg.gridDimX, cfg.gridDimY, cfg.gridDimZ,
									 cfg.blockDimX, cfg.blockDimY, cfg.blockDimZ, cfg.sharedMemBytes, stream, op->op_args, NULL),
			   "hipModuleLaunchKernel", {
			fprintf(stderr, "Error: failed to launch kernel for op with nickname %s...\n", op->op_skeleton.header.op_nickname);
			return -1; });
		return 0;
	}
	if (!fn->hip_external_func) {
		fprintf(stderr, "Error: if op is not native it must have a reference to external function (error with op having nickname %s)\n", op->op_skeleton.header.op_nickname);
		return -1;
	}
	if ((fn->hip_external_func)(h, stream_id, op, fn->op_extra)) {
		fprintf(stderr, "Error: failed to do external function for op with nickname %s...\n", op->op_skeleton.header.op_nickname);
		return -1;
	}
	return 0;
}

static int hip_submit_host_op(Dataflow_Handle * h, void * host_func, void * host_func_arg, int stream_id) {
	hipStream_t stream;
	if (resolve_stream(h, stream_id, &stream, "submit host op") || make_current(h)) {
		return -1;
	}
	HIP_OK(hipLaunchHostFunc(stream, (hipHostFn_t) host_func, host_func_arg), "hipLaunchHostFunc", return -1);
	return 0;
}

/* ------------------------------------------------------------------ dependencies */

static void * hip_get_stream_state(Dataflow_Handle * h, int stream_id) {
	if (stream_id < 0 || stream_id >= h->num_streams) {
		fprintf(stderr, "Error: cannot get stream state for stream id %d, when device only has %d streams...\n", stream_id, h->num_streams);
		return NULL;
	}
	if (make_current(h)) {
		return NULL;
	}
	hipEvent_t * ev = &(handle_events(h)[stream_id]);
	HIP_OK(hipEventRecord(*ev, handle_streams(h)[stream_id]), "hipEventRecord", return NULL);
	return (void *) ev;
}

static int hip_submit_dependency(Dataflow_Handle * h, int stream_id, void * other_stream_state) {
	hipStream_t stream;
	if (!other_stream_state) {
		fprintf(stderr, "Error: cannot submit dependency on a NULL stream state...\n");
		return -1;
	}
	if (resolve_stream(h, stream_id, &stream, "submit dependency") || make_current(h)) {
		return -1;
	}
	HIP_OK(hipStreamWaitEvent(stream, *((hipEvent_t *) other_stream_state), 0), "hipStreamWaitEvent", return -1);
	return 0;
}

static int hip_sync_stream(Dataflow_Handle * h, int stream_id) {
	hipStream_t stream;
	if (resolve_stream(h, stream_id, &stream, "sync stream") || make_current(h)) {
		return -1;
	}
	HIP_OK(hipStreamSynchronize(stream), "hipStreamSynchronize", return -1);
	return 0;
}

static int hip_sync_handle(Dataflow_Handle * h) {
	if (make_current(h)) {
		return -1;
	}
	HIP_OK(hipDeviceSynchronize(), "hipDeviceSynchronize", return -1);
	return 0;
}

/* ------------------------------------------------------------------ memory */

static void * hip_alloc_mem(Dataflow_Handle * h, uint64_t size_bytes) {
	if (make_current(h)) {
		return NULL;
	}
	void * p = NULL;
	HIP_OK(hipMalloc(&p, (size_t) size_bytes), "hipMalloc", return NULL);
	return p;
}

static void hip_free_mem(Dataflow_Handle * h, void * dev_ptr) {
	if (!dev_ptr || make_current(h)) {
		return;
	}
	HIP_OK(hipFree(dev_ptr), "hipFree", return);
}

static int hip_set_mem(Dataflow_Handle * h, int stream_id, void * dev_ptr, uint8_t val, uint64_t size_bytes) {
	if (make_current(h)) {
		return -1;
	}
	if (size_bytes == 0) {
		return 0;
	}
	if (stream_id == -1) {
		HIP_OK(hipMemset(dev_ptr, (int) val, (size_t) size_bytes), "hipMemset", return -1);
		return 0;
	}
	hipStream_t stream;
	if (resolve_stream(h, stream_id, &stream, "set mem")) {
		return -1;
	}
	HIP_OK(hipMemsetD8Async((hipDeviceptr_t) dev_ptr, val, (size_t) size_bytes, stream), "hipMemsetD8Async", return -1);
	return 0;
}

/* 1 if the `size_bytes` bytes at `host_ptr` lie in one piece of page-locked host memory that the device can already
 * address (hipHostMalloc, i.e. dataflow_amd_alloc_host_mem), 0 if not.  First and last byte must both be such memory,
 * and where the runtime tells the extent of the allocation the range must end inside it. */
static int host_mem_is_device_visible(void * host_ptr, uint64_t size_bytes) {
	hipPointerAttribute_t first, last;
	memset(&first, 0, sizeof(first));
	memset(&last, 0, sizeof(last));
	if (hipPointerGetAttributes(&first, host_ptr) != hipSuccess) {
		(void) hipGetLastError();                     /* a plain pointer is "invalid value" to the query: not an error of ours */
		return 0;
	}
	if (first.type != hipMemoryTypeHost) {
		return 0;
	}
	if (size_bytes <= 1) {
		return 1;
	}
	if (hipPointerGetAttributes(&last, (uint8_t *) host_ptr + size_bytes - 1) != hipSuccess) {
		(void) hipGetLastError();
		return 0;
	}
	if (last.type != hipMemoryTypeHost) {
		return 0;
	}
	hipDeviceptr_t base = NULL;
	size_t extent = 0;
	if (first.devicePointer && hipMemGetAddressRange(&base, &extent, (hipDeviceptr_t) first.devicePointer) == hipSuccess) {
		const uint64_t offset = (uint64_t) ((uint8_t *) first.devicePointer - (uint8_t *) base);
		return offset + size_bytes <= (uint64_t) extent;
	}
	(void) hipGetLastError();
	return 1;
}

/* The reference pins memory that already exists (cuMemHostRegister, cuda_dataflow_handle.c:604-620).  Registering
 * existing pages is not supported by this backend: the driver refuses it on some systems and leaves an error
 * behind that the next, unrelated call reports.  So the call never registers anything: memory that came from
 * dataflow_amd_alloc_host_mem is already visible to the device and is accepted (0); anything else is refused (-1)
 * with a message that names the allocator to use; so is a range that runs past the end of such an allocation. */
static int hip_enable_access_to_host_mem(Dataflow_Handle * h, void * host_ptr, uint64_t size_bytes, unsigned int flags) {
	(void) flags;
	if (!host_ptr || make_current(h)) {
		return -1;
	}
	if (host_mem_is_device_visible(host_ptr, size_bytes)) {
		return 0;
	}
	fprintf(stderr, "Error: this backend does not pin existing host memory (%lu bytes at %p). Allocate device-visible host memory with dataflow_amd_alloc_host_mem instead...\n",
			(unsigned long) size_bytes, host_ptr);
	return -1;
}

/* the counterpart: nothing was registered, so there is nothing to undo for memory of dataflow_amd_alloc_host_mem
 * (it stays visible until dataflow_amd_free_host_mem); any other pointer was never enabled and is an error */
static int hip_disable_access_to_host_mem(Dataflow_Handle * h, void * host_ptr) {
	if (!host_ptr || make_current(h)) {
		return -1;
	}
	if (host_mem_is_device_visible(host_ptr, 1)) {
		return 0;
	}
	fprintf(stderr, "Error: disable_access_to_host_mem on memory that was never made visible to the device (%p)...\n", host_ptr);
	return -1;
}

static int hip_enable_access_to_peer_mem(Dataflow_Handle * h, Dataflow_Handle * peer) {
	if (!peer || make_current(h)) {
		return -1;
	}
	if (peer->device_id == h->device_id) {
		return 0;
	}
	hipError_t e = hipDeviceEnablePeerAccess(peer->device_id, 0);
	if (e != hipSuccess && e != hipErrorPeerAccessAlreadyEnabled) {
		(void) hipGetLastError();
		fprintf(stderr, "Error: could not enable peer access from device %d to %d: %s...\n", h->device_id, peer->device_id, hipGetErrorString(e));
		return -1;
	}
	(void) hipGetLastError();
	return 0;
}

static int hip_disable_access_to_peer_mem(Dataflow_Handle * h, Dataflow_Handle * peer) {
	if (!peer || make_current(h)) {
		return -1;
	}
	if (peer->device_id == h->device_id) {
		return 0;
	}
	hipError_t e = hipDeviceDisablePeerAccess(peer->device_id);
	if (e != hipSuccess) {
		(void) hipGetLastError();
		fprintf(stderr, "Error: could not disable peer access from device %d to %d: %s...\n", h->device_id, peer->device_id, hipGetErrorString(e));
		return -1;
	}
	return 0;
}

/* ------------------------------------------------------------------ transfers */

static int do_copy(Dataflow_Handle * h, int stream_id, void * dst, void * src, uint64_t size_bytes, hipMemcpyKind kind, const char * what) {
	hipStream_t stream;
	if (resolve_stream(h, stream_id, &stream, what) || make_current(h)) {
		return -1;
	}
	if (size_bytes == 0) {
		return 0;
	}
	HIP_OK(hipMemcpyAsync(dst, src, (size_t) size_bytes, kind, stream), what, return -1);
	return 0;
}

static int hip_submit_inbound_transfer(Dataflow_Handle * h, int stream_id, void * dev_dest, void * host_src, uint64_t size_bytes) {
	return do_copy(h, stream_id, dev_dest, host_src, size_bytes, hipMemcpyHostToDevice, "submit inbound transfer");
}
static int hip_submit_outbound_transfer(Dataflow_Handle * h, int stream_id, void * host_dest, void * dev_src, uint64_t size_bytes) {
	return do_copy(h, stream_id, host_dest, dev_src, size_bytes, hipMemcpyDeviceToHost, "submit outbound transfer");
}
static int hip_submit_peer_transfer(Dataflow_Handle * h, int stream_id, void * dev_dest, void * dev_src, uint64_t size_bytes) {
	return do_copy(h, stream_id, dev_dest, dev_src, size_bytes, hipMemcpyDeviceToDevice, "submit peer transfer");
}

/* ------------------------------------------------------------------ init / destroy */

int dataflow_init_handle(Dataflow_Handle * h, ComputeType compute_type, int device_id, int ctx_id, unsigned int ctx_flags,
						 int num_streams, int * opt_stream_prios, char ** opt_stream_names, float compute_frac) {
	(void) ctx_flags;
	if (!h) {
		fprintf(stderr, "Error: dataflow_init_handle needs a handle to fill...\n");
		return -1;
	}
	if (compute_type != COMPUTE_HSA) {
		fprintf(stderr, "Error: this backend only implements COMPUTE_HSA (%d), got compute type %d...\n", (int) COMPUTE_HSA, (int) compute_type);
		return -1;
	}
	if (num_streams < 1 || num_streams > MAX_STREAMS) {
		fprintf(stderr, "Error: number of streams must be in [1, %d], got %d...\n", MAX_STREAMS, num_streams);
		return -1;
	}
	if (compute_frac > 0.0f && compute_frac < 1.0f) {
		fprintf(stderr, "Warning: compute_frac %.3f ignored; this backend always uses every compute unit...\n", compute_frac);
	}
	memset(h, 0, sizeof(*h));

	int dev_count = 0;
	HIP_OK(hipGetDeviceCount(&dev_count), "hipGetDeviceCount", return -1);
	if (device_id < 0 || device_id >= dev_count) {
		fprintf(stderr, "Error: device id %d out of range, %d devices visible...\n", device_id, dev_count);
		return -1;
	}
	HIP_OK(hipSetDevice(device_id), "hipSetDevice", return -1);

	hipDeviceProp_t prop;
	HIP_OK(hipGetDeviceProperties(&prop, device_id), "hipGetDeviceProperties", return -1);

	Hip_Device_Info * info = (Hip_Device_Info *) calloc(1, sizeof(Hip_Device_Info));
	if (!info) {
		fprintf(stderr, "Error: malloc failed for device info...\n");
		return -1;
	}
	info->total_mem = prop.totalGlobalMem;
	info->cu_count = prop.multiProcessorCount;
	info->wavefront_size = prop.warpSize;
	info->max_threads_per_block = prop.maxThreadsPerBlock;
	info->max_lds_per_block = (int) prop.sharedMemPerBlock;
	info->optin_max_lds_per_block = (int) prop.sharedMemPerBlockOptin ? (int) prop.sharedMemPerBlockOptin : (int) prop.sharedMemPerBlock;
	info->clock_khz = prop.clockRate;
	info->host_numa_id = -1;
	snprintf(info->device_name, sizeof(info->device_name), "%s", prop.name);
	snprintf(info->arch_name, sizeof(info->arch_name), "%s", prop.gcnArchName);
	int arch = 0;
	if (sscanf(prop.gcnArchName, "gfx%d", &arch) == 1) {
		info->arch_num = arch;
	}
	/* CDNA3/4 parts expose 8 accelerator complex dies; work-groups are dealt to them round-robin */
	info->xcd_count = (arch == 942 || arch == 950) ? 8 : 1;

	h->compute_type = COMPUTE_HSA;
	h->device_id = device_id;
	h->device_handle = NULL;
	h->device_info = info;
	h->hardware_arch_type = UNKNOWN_HARDWARE_ARCH;
	h->pcie_link_width = 0;
	h->pcie_link_gen = 0;
	h->ctx_id = ctx_id;
	h->ctx = NULL;
	h->num_streams = num_streams;

	hipStream_t * streams = (hipStream_t *) calloc((size_t) num_streams, sizeof(hipStream_t));
	hipEvent_t * events = (hipEvent_t *) calloc((size_t) num_streams, sizeof(hipEvent_t));
	if (!streams || !events) {
		fprintf(stderr, "Error: malloc failed for stream containers...\n");
		free(streams); free(events); free(info);
		return -1;
	}
	for (int i = 0; i < num_streams; i++) {
		HIP_OK(hipStreamCreateWithFlags(&streams[i], hipStreamNonBlocking), "hipStreamCreateWithFlags", return -1);
		HIP_OK(hipEventCreateWithFlags(&events[i], hipEventDisableTiming), "hipEventCreateWithFlags", return -1);
		h->stream_prios[i] = opt_stream_prios ? opt_stream_prios[i] : 0;
		h->stream_names[i] = (opt_stream_names && opt_stream_names[i]) ? strdup(opt_stream_names[i]) : NULL;
	}
	h->streams = streams;
	h->stream_states = events;

	h->num_native_function_libs = 0;
	h->num_ops = 0;
	if (dataflow_init_table(&h->op_table, hip_op_table_hash_func, DATAFLOW_OP_IDENTIFIER_FINGERPRINT_NUM_BYTES, sizeof(Hip_Function),
							OP_TABLE_MIN_SIZE, OP_TABLE_MAX_SIZE, 0.5f, 0.1f)) {
		fprintf(stderr, "Error: failed to init op table...\n");
		return -1;
	}

	h->profiler.start = hip_profiler_start;
	h->profiler.stop = hip_profiler_stop;
	h->profiler.name_device = hip_profiler_name_device;
	h->profiler.name_handle = hip_profiler_name_handle;
	h->profiler.name_stream = hip_profiler_name_stream;
	h->profiler.name_thread = hip_profiler_name_thread;
	h->profiler.range_push = hip_profiler_range_push;
	h->profiler.range_pop = hip_profiler_range_pop;

	h->get_num_procs = hip_get_num_procs;
	h->register_native_code = hip_register_native_code;
	h->register_external_code = hip_register_external_code;
	h->submit_op = hip_submit_op;
	h->submit_host_op = hip_submit_host_op;
	h->get_stream_state = hip_get_stream_state;
	h->submit_dependency = hip_submit_dependency;
	h->sync_stream = hip_sync_stream;
	h->sync_handle = hip_sync_handle;
	h->alloc_mem = hip_alloc_mem;
	h->free_mem = hip_free_mem;
	h->set_mem = hip_set_mem;
	h->enable_access_to_host_mem = hip_enable_access_to_host_mem;
	h->disable_access_to_host_mem = hip_disable_access_to_host_mem;
	h->enable_access_to_peer_mem = hip_enable_access_to_peer_mem;
	h->disable_access_to_peer_mem = hip_disable_access_to_peer_mem;
	h->submit_inbound_transfer = hip_submit_inbound_transfer;
	h->submit_outbound_transfer = hip_submit_outbound_transfer;
	h->submit_peer_transfer = hip_submit_peer_transfer;
	return 0;
}

void * dataflow_amd_alloc_host_mem(Dataflow_Handle * h, uint64_t size_bytes) {
	if (!h || make_current(h)) {
		return NULL;
	}
	void * p = NULL;
	HIP_OK(hipHostMalloc(&p, (size_t) size_bytes, hipHostMallocPortable | hipHostMallocMapped), "hipHostMalloc", return NULL);
	return p;
}

void dataflow_amd_free_host_mem(Dataflow_Handle * h, void * host_ptr) {
	if (!h || !host_ptr || make_current(h)) {
		return;
	}
	HIP_OK(hipHostFree(host_ptr), "hipHostFree", return);
}

void * dataflow_amd_get_stream(Dataflow_Handle * h, int stream_id) {
	if (!h || stream_id < 0 || stream_id >= h->num_streams) {
		return NULL;
	}
	return (void *) handle_streams(h)[stream_id];
}

void dataflow_amd_destroy_handle(Dataflow_Handle * h) {
	if (!h || !h->streams) {
		return;
	}
	if (make_current(h)) {
		return;
	}
	(void) hipDeviceSynchronize();
	/* external libraries may hold per-op state; give each a chance to release it */
	for (int i = 0; i < h->num_streams; i++) {
		(void) hipStreamDestroy(handle_streams(h)[i]);
		(void) hipEventDestroy(handle_events(h)[i]);
		free(h->stream_names[i]);
		h->stream_names[i] = NULL;
	}
	for (int i = 0; i < h->num_native_function_libs; i++) {
		(void) hipModuleUnload((hipModule_t) h->native_function_libs[i]);
	}
	dataflow_destroy_table(&h->op_table);
	free(h->streams);
	free(h->stream_states);
	free(h->device_info);
	h->streams = NULL;
	h->stream_states = NULL;
	h->device_info = NULL;
	h->num_streams = 0;
	h->num_ops = 0;
	h->num_native_function_libs = 0;
}
