/*
 * dataflow_amd.h -- the C boundary of the gfx950 MoE backend.
 *
 * Everything a caller of ml_dataflow's backend interface sees is restated here so that
 * this backend can be built with no file of the reference on the include path, while a
 * program compiled against the reference's own headers can still hand its
 * Dataflow_Handle / Op structs to this library: all struct layouts, enum values and
 * function-pointer signatures below are byte-compatible with
 *
 *   libdataflow/include/dataflow_common.h:50-93        (DataflowDatatype, fingerprint size)
 *   libdataflow/include/dataflow_op_structs.h:6-30     (Op_Skeleton_Header, Op_Skeleton, Op)
 *   libdataflow/include/dataflow_table.h:31-71         (Table_Config, Dataflow_Table)
 *   libdataflow/include/dataflow_handle.h:9-166        (ComputeType, Dataflow_Profiler, Dataflow_Handle,
 *                                                       External_Lib_Func, External_Lib_Func_Init)
 *   libdataflow/include/dataflow.h:11                  (dataflow_init_handle)
 *   backends/nvidia/include/register_ops.h:8           (dataflow_register_default_ops)
 *
 * Error convention everywhere (same as the reference): int functions return 0 on
 * success and -1 on error with a message on stderr; pointer functions return NULL.
 */
#ifndef DATAFLOW_AMD_H
#define DATAFLOW_AMD_H

#include <stdint.h>
#include <stddef.h>
#include <stdbool.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- element / scalar type tags (dataflow_common.h:50-79) ---- */
typedef enum {
	DATAFLOW_NONE,
	DATAFLOW_VOID,
	DATAFLOW_FP64,
	DATAFLOW_FP32,
	DATAFLOW_FP16,
	DATAFLOW_BF16,
	DATAFLOW_FP8E4M3,
	DATAFLOW_FP8E5M2,
	DATAFLOW_UINT64,
	DATAFLOW_UINT32,
	DATAFLOW_UINT16,
	DATAFLOW_UINT8,
	DATAFLOW_LONG,
	DATAFLOW_INT,
	DATAFLOW_BOOL,
	DATAFLOW_FP64_SCALAR,
	DATAFLOW_FP32_SCALAR,
	DATAFLOW_FP16_SCALAR,
	DATAFLOW_BF16_SCALAR,
	DATAFLOW_FP8E4M3_SCALAR,
	DATAFLOW_FP8E5M2_SCALAR,
	DATAFLOW_UINT64_SCALAR,
	DATAFLOW_UINT32_SCALAR,
	DATAFLOW_UINT16_SCALAR,
	DATAFLOW_UINT8_SCALAR,
	DATAFLOW_LONG_SCALAR,
	DATAFLOW_INT_SCALAR,
	DATAFLOW_BOOL_SCALAR
} DataflowDatatype;

#define DATAFLOW_OP_IDENTIFIER_FINGERPRINT_TYPE 0        /* SHA-256 */
#define DATAFLOW_OP_IDENTIFIER_FINGERPRINT_NUM_BYTES 32

/* ---- op identity and argument carrier (dataflow_op_structs.h) ---- */
#define MAX_OP_ARGS 32
#define MAX_OP_NICKNAME_SIZE 255

/* 256 + 4 + 32*4 = 388 bytes, no padding: the fingerprint is SHA-256 over exactly these bytes. */
typedef struct op_skeleton_header {
	char op_nickname[MAX_OP_NICKNAME_SIZE + 1];
	int num_args;
	DataflowDatatype arg_dtypes[MAX_OP_ARGS];
} Op_Skeleton_Header;

typedef struct op_identifier {
	uint8_t fingerprint[DATAFLOW_OP_IDENTIFIER_FINGERPRINT_NUM_BYTES];
} Op_Identifier;

typedef struct Op_Skeleton {
	Op_Skeleton_Header header;
	Op_Identifier identifier;
} Op_Skeleton;

/* op_args[i] points at the VALUE of argument i (also for pointer arguments: op_args[i] = &ptr).
 * The storage is only valid for the duration of submit_op. */
typedef struct op {
	Op_Skeleton op_skeleton;
	void * op_args[MAX_OP_ARGS];
} Op;

/* ---- open-addressing table that lives by value inside the handle (dataflow_table.h) ---- */
typedef uint64_t (*Hash_Func)(void * item, uint64_t table_size);

typedef struct table_config {
	uint64_t min_size;
	uint64_t max_size;
	float load_factor;
	float shrink_factor;
	Hash_Func hash_func;
	uint64_t key_size_bytes;
	uint64_t value_size_bytes;
} Table_Config;

typedef struct table {
	uint64_t cnt;
	uint64_t size;
	Table_Config config;
	uint64_t * is_empty_bit_vector;
	void * items;
} Dataflow_Table;

/* ---- the handle (dataflow_handle.h) ---- */
#define OP_TABLE_MIN_SIZE 1UL << 10
#define OP_TABLE_MAX_SIZE 1UL << 20
#define MAX_NATIVE_FUNCTION_LIBS 1024
#define MAX_STREAMS 256
#define FUNC_SYMBOL_MAX_LEN 512

typedef enum compute_type {
	COMPUTE_NONE,
	COMPUTE_CPU,
	COMPUTE_CUDA,
	COMPUTE_HSA,          /* the value this backend accepts */
	COMPUTE_LEVEL_ZERO
} ComputeType;

typedef enum hardware_arch_type {
	BACKEND_ARCH_A100,
	BACKEND_ARCH_RTX_3090,
	BACKEND_ARCH_RTX_4090,
	BACKEND_ARCH_RTX_5090,
	BACKEND_ARCH_H100,
	UNKNOWN_HARDWARE_ARCH   /* what this backend reports: the enum has no AMD entry */
} HardwareArchType;

typedef struct dataflow_handle Dataflow_Handle;

typedef struct dataflow_profiler {
	int (*start)(void);
	int (*stop)(void);
	void (*name_device)(Dataflow_Handle * dataflow_handle, const char * device_name);
	void (*name_handle)(Dataflow_Handle * dataflow_handle, const char * handle_name);
	void (*name_stream)(Dataflow_Handle * dataflow_handle, int stream_id, const char * stream_name);
	void (*name_thread)(Dataflow_Handle * dataflow_handle, const char * thread_name);
	int (*range_push)(const char * message);
	int (*range_pop)(void);
} Dataflow_Profiler;

struct dataflow_handle {
	Dataflow_Profiler profiler;
	ComputeType compute_type;
	int device_id;
	void * device_handle;
	void * device_info;                 /* -> Hip_Device_Info for this backend */
	HardwareArchType hardware_arch_type;
	unsigned int pcie_link_width;
	unsigned int pcie_link_gen;
	int ctx_id;
	void * ctx;
	int num_streams;
	void * streams;                     /* hipStream_t[num_streams] */
	int stream_prios[MAX_STREAMS];
	char * stream_names[MAX_STREAMS];
	void * stream_states;               /* hipEvent_t[num_streams], one re-recorded event per stream */
	int num_native_function_libs;
	void * native_function_libs[MAX_NATIVE_FUNCTION_LIBS];
	int num_ops;
	Dataflow_Table op_table;            /* fingerprint -> Hip_Function */

	int (*get_num_procs)(Dataflow_Handle * dataflow_handle);

	int (*register_native_code)(Dataflow_Handle * dataflow_handle, char * native_code_filename,
								char * native_code_config_lib_filename, int num_funcs,
								Op_Skeleton * func_op_skeletons, char ** func_symbols,
								char ** func_set_launch_symbols, char ** func_init_symbols);
	int (*register_external_code)(Dataflow_Handle * dataflow_handle, char * external_code_filename, int num_funcs,
								Op_Skeleton * func_op_skeletons, char ** func_symbols, char ** func_init_symbols);

	int (*submit_op)(Dataflow_Handle * dataflow_handle, Op * op, int stream_id);
	int (*submit_host_op)(Dataflow_Handle * dataflow_handle, void * host_func, void * host_func_arg, int stream_id);

	void * (*get_stream_state)(Dataflow_Handle * dataflow_handle, int stream_id);
	int (*submit_dependency)(Dataflow_Handle * dataflow_handle, int stream_id, void * other_stream_state);
	int (*sync_stream)(Dataflow_Handle * dataflow_handle, int stream_id);
	int (*sync_handle)(Dataflow_Handle * dataflow_handle);

	void * (*alloc_mem)(Dataflow_Handle * dataflow_handle, uint64_t size_bytes);
	void (*free_mem)(Dataflow_Handle * dataflow_handle, void * dev_ptr);
	int (*set_mem)(Dataflow_Handle * dataflow_handle, int stream_id, void * dev_ptr, uint8_t val, uint64_t size_bytes);
	int (*enable_access_to_host_mem)(Dataflow_Handle * dataflow_handle, void * host_ptr, uint64_t size_bytes, unsigned int flags);
	int (*disable_access_to_host_mem)(Dataflow_Handle * dataflow_handle, void * host_ptr);
	int (*enable_access_to_peer_mem)(Dataflow_Handle * dataflow_handle, Dataflow_Handle * peer_dataflow_handle);
	int (*disable_access_to_peer_mem)(Dataflow_Handle * dataflow_handle, Dataflow_Handle * peer_dataflow_handle);

	int (*submit_inbound_transfer)(Dataflow_Handle * dataflow_handle, int stream_id, void * dev_dest, void * host_src, uint64_t size_bytes);
	int (*submit_outbound_transfer)(Dataflow_Handle * dataflow_handle, int stream_id, void * host_dest, void * dev_src, uint64_t size_bytes);
	int (*submit_peer_transfer)(Dataflow_Handle * dataflow_handle, int stream_id, void * dev_dest, void * dev_src, uint64_t size_bytes);
};

/* signatures of code registered through register_external_code (dataflow_handle.h:161,166) */
typedef int (*External_Lib_Func_Init)(Dataflow_Handle * dataflow_handle, void * op_table_value);
typedef int (*External_Lib_Func)(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra);

/* ---- what this backend stores behind the opaque pointers ---- */

/* dataflow_handle->device_info. Counterpart of Cuda_Device_Info (backends/nvidia/include/cuda_dataflow_handle.h:16-27). */
typedef struct hip_device_info {
	size_t total_mem;
	int arch_num;                     /* 950 for gfx950 */
	int cu_count;                     /* compute units; reported by get_num_procs */
	int xcd_count;                    /* accelerator complex dies (8 on MI355X) */
	int wavefront_size;               /* 64 */
	int max_threads_per_block;
	int max_lds_per_block;            /* static limit */
	int optin_max_lds_per_block;      /* with hipFuncAttributeMaxDynamicSharedMemorySize */
	int clock_khz;
	int host_numa_id;
	char device_name[256];
	char arch_name[64];               /* "gfx950..." */
} Hip_Device_Info;

/* grid/block/LDS of one native launch. Counterpart of Cuda_Launch_Config (cuda_dataflow_handle.h:34-42). */
typedef struct hip_launch_config {
	unsigned int gridDimX;
	unsigned int gridDimY;
	unsigned int gridDimZ;
	unsigned int blockDimX;
	unsigned int blockDimY;
	unsigned int blockDimZ;
	unsigned int sharedMemBytes;
} Hip_Launch_Config;

typedef struct hip_function_config {
	int func_max_lds;
	int func_max_threads_per_block;
} Hip_Function_Config;

typedef struct hip_function Hip_Function;

/* value type of the op table. Counterpart of Cuda_Function (cuda_dataflow_handle.h:47-64). */
struct hip_function {
	Hip_Function_Config function_config;
	bool is_native;
	void * function_handle;           /* hipFunction_t when native */
	int (*set_launch_config)(Hip_Launch_Config * launch_config, Dataflow_Handle * dataflow_handle, Hip_Function * hip_function, Op * op);
	int (*hip_external_func)(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra);
	void * op_extra;
	Op_Skeleton op_skeleton;
};

/* optional per-kernel attribute hook looked up in the launch-config library (cuda_dataflow_handle.h:66) */
typedef int (*Hip_Set_Func_Attribute)(Dataflow_Handle * dataflow_handle, Hip_Function * hip_function);

/* ---- exported entry points ---- */

/* Replaces cuda_dataflow_handle.c:865 dataflow_init_handle. compute_type must be COMPUTE_HSA.
 * Stream priorities are accepted but every stream is created at the default priority. */
int dataflow_init_handle(Dataflow_Handle * dataflow_handle, ComputeType compute_type, int device_id, int ctx_id,
						 unsigned int ctx_flags, int num_streams, int * opt_stream_prios, char ** opt_stream_names,
						 float compute_frac);

/* Replaces register_ops.c:412 dataflow_register_default_ops. Registers the ops of the MoE layer, the RMS norm around it, the AdamW step and the two
 * casts only (bf16; select_experts also for fp32 logits, swiglu and swiglu_bwd_x also for fp32 and fp16 elements, the
 * other element types the reference has real kernels for on this path) and returns how many were added
 * (DATAFLOW_AMD_NUM_DEFAULT_OPS) or -1. Code objects are looked up in
 * $DATAFLOW_AMD_LIB_DIR, else next to the shared library that contains this function. */
int dataflow_register_default_ops(Dataflow_Handle * dataflow_handle);
#define DATAFLOW_AMD_NUM_DEFAULT_OPS 31

/* libdataflow utilities (dataflow.h:18-61) */
size_t dataflow_sizeof_element(DataflowDatatype arr_dtype);
char * dataflow_datatype_as_string(DataflowDatatype dtype);
int dataflow_do_fingerprinting(void * data, uint64_t num_bytes, uint8_t * ret_fingerprint);
int dataflow_init_table(Dataflow_Table * table, Hash_Func hash_func, uint64_t key_size_bytes, uint64_t value_size_bytes,
						uint64_t min_table_size, uint64_t max_table_size, float load_factor, float shrink_factor);
void dataflow_destroy_table(Dataflow_Table * table);
int dataflow_insert_table(Dataflow_Table * table, void * key, void * value);
long dataflow_find_table(Dataflow_Table * table, void * key, bool to_copy_value, void ** ret_value);
int dataflow_remove_table(Dataflow_Table * table, void * key, void * ret_value);

/* scalar bf16 helpers (dataflow_common.h:81-92); fp32->bf16 is round-to-nearest-even here */
float solo_bf16_to_fp32(uint16_t a);
uint16_t solo_fp32_to_bf16(float f);

/* ---- additions with no counterpart in the reference ---- */

/* Page-locked, device-visible host memory (hipHostMalloc). The reference pins existing memory through
 * enable_access_to_host_mem; where the driver refuses to register existing pages, callers that need a
 * device-writable host buffer (host_expert_counts) allocate it here instead. */
void * dataflow_amd_alloc_host_mem(Dataflow_Handle * dataflow_handle, uint64_t size_bytes);
void dataflow_amd_free_host_mem(Dataflow_Handle * dataflow_handle, void * host_ptr);
/* releases streams, events, modules, the op table and device_info */
void dataflow_amd_destroy_handle(Dataflow_Handle * dataflow_handle);
/* raw hipStream_t of a stream id (for callers that time with HIP events), NULL if out of range */
void * dataflow_amd_get_stream(Dataflow_Handle * dataflow_handle, int stream_id);

#ifdef __cplusplus
}
#endif

#endif
