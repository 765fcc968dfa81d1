/*
 * moe_files.c -- the reference's on-disk formats as far as the MoE layer meets them (see include/moe_layer.h):
 *
 *   layers/<i>/combined_layer.weight   every weight of one transformer block back to back, written by
 *                                      models/init_model.py:205-318 and read whole by
 *                                      libdataflowmodels/src/transformer/src/prep_transformer.c:366-388 into a buffer
 *                                      laid out by set_transformer_block_weight_offsets (:24-165);
 *   <dir>/layers_fwd/<i>/seq_<s>_chunk_<c>_<name>.dat   raw arrays saved for inspection by save_file
 *                                      (dataflow_transformer.c:46-160), read back by the reference's
 *                                      test/dataflow_models/correctness_compare scripts.
 *
 * Host code only: plain stdio plus the handle's transfers.
 */
#define _FILE_OFFSET_BITS 64
#include "moe_layer.h"

#include <sys/types.h>
#include <errno.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* prep_transformer.c:3-20: an array starts at the running aligned size, which then grows by the array's size and
 * is rounded up to the alignment */
static void place(uint64_t * offset, uint64_t size, uint64_t * raw, uint64_t * aligned, int alignment) {
	*offset = *aligned;
	*raw += size;
	*aligned += size;
	if (alignment > 0 && (*aligned % (uint64_t) alignment) > 0) {
		*aligned += (uint64_t) alignment - (*aligned % (uint64_t) alignment);
	}
}

int amd_moe_block_weight_offsets(int model_dim, int attn_dim, int kv_dim, int num_experts, int expert_dim,
								 DataflowDatatype dt, int pointer_alignment, Amd_Moe_Block_Offsets * out) {
	uint64_t el = (uint64_t) dataflow_sizeof_element(dt);
	if (!out || el == 0 || model_dim < 1 || attn_dim < 0 || kv_dim < 0 || num_experts < 1 || expert_dim < 1 || pointer_alignment < 0) {
		fprintf(stderr, "Error: cannot set block weight offsets (model_dim=%d attn_dim=%d kv_dim=%d experts=%d expert_dim=%d dtype=%s)...\n",
				model_dim, attn_dim, kv_dim, num_experts, expert_dim, dataflow_datatype_as_string(dt));
		return -1;
	}
	memset(out, 0, sizeof(*out));
	uint64_t D = (uint64_t) model_dim, A = (uint64_t) attn_dim, KV = (uint64_t) kv_dim, H = (uint64_t) expert_dim;
	uint64_t raw = 0, aligned = 0;
	/* order and sizes: prep_transformer.c:140-159 (exact attention, RMS norm, MoE MLP; the router is stored in the
	 * block's element type, :94-96) */
	place(&out->w_attn_norm, D * el, &raw, &aligned, pointer_alignment);
	place(&out->w_q, D * A * el, &raw, &aligned, pointer_alignment);
	place(&out->w_k, D * KV * el, &raw, &aligned, pointer_alignment);
	place(&out->w_v, D * KV * el, &raw, &aligned, pointer_alignment);
	place(&out->w_o, A * D * el, &raw, &aligned, pointer_alignment);
	place(&out->w_ffn_norm, D * el, &raw, &aligned, pointer_alignment);
	place(&out->w_router, D * (uint64_t) num_experts * el, &raw, &aligned, pointer_alignment);
	uint64_t w1, w3, w2, prev_w1 = 0;
	for (int e = 0; e < num_experts; e++) {
		place(&w1, D * H * el, &raw, &aligned, pointer_alignment);
		place(&w3, D * H * el, &raw, &aligned, pointer_alignment);
		place(&w2, H * D * el, &raw, &aligned, pointer_alignment);
		if (e == 0) {
			out->w_1 = w1;
			out->w_3 = w3;
			out->w_2 = w2;
		} else if (e == 1) {
			out->expert_stride = w1 - prev_w1;
		}
		prev_w1 = w1;
	}
	if (num_experts == 1) {
		out->expert_stride = aligned - out->w_1;
	}
	out->raw_size = raw;
	out->aligned_size = aligned;
	return 0;
}

static int read_at(FILE * file, const char * filename, uint64_t offset, void * dst, uint64_t bytes) {
	if (fseeko(file, (off_t) offset, SEEK_SET) != 0) {
		fprintf(stderr, "Error: could not seek to byte %lu of %s: %s...\n", (unsigned long) offset, filename, strerror(errno));
		return -1;
	}
	size_t got = fread(dst, 1, bytes, file);
	if (got != bytes) {
		fprintf(stderr, "Error: could not read file %s. Expected %lu bytes at offset %lu, but read %zu bytes...\n",
				filename, (unsigned long) bytes, (unsigned long) offset, got);
		return -1;
	}
	return 0;
}

int amd_moe_layer_load_block_file(Dataflow_Handle * handle, int stream_id, Amd_Moe_Layer * layer, const char * filename,
								  int attn_dim, int kv_dim, int pointer_alignment, void * ffn_norm_weight) {
	if (!handle || !layer || !filename || !layer->w_router || !layer->w1 || !layer->w3 || !layer->w2) {
		fprintf(stderr, "Error: cannot load a block file into an unallocated layer...\n");
		return -1;
	}
	Amd_Moe_Block_Offsets off;
	if (amd_moe_block_weight_offsets(layer->model_dim, attn_dim, kv_dim, layer->num_experts, layer->expert_dim, layer->dt,
									 pointer_alignment, &off)) {
		return -1;
	}
	FILE * file = fopen(filename, "rb");
	if (!file) {
		fprintf(stderr, "Error: could not open file %s...\n", filename);
		return -1;
	}
	/* the reference reads block_aligned_size bytes in one piece and fails on a shorter file (prep_transformer.c:378-383) */
	if (fseeko(file, 0, SEEK_END) != 0 || (uint64_t) ftello(file) < off.aligned_size) {
		fprintf(stderr, "Error: could not read file %s. Expected %lu bytes (aligned size), but the file is shorter...\n",
				filename, (unsigned long) off.aligned_size);
		fclose(file);
		return -1;
	}
	const uint64_t el = (uint64_t) dataflow_sizeof_element(layer->dt);
	const uint64_t D = (uint64_t) layer->model_dim, H = (uint64_t) layer->expert_dim, E = (uint64_t) layer->num_experts;
	const uint64_t up = D * H * el;
	const uint64_t router = D * E * el;
	uint64_t staging_bytes = 3 * up > router ? 3 * up : router;
	uint8_t * staging = (uint8_t *) malloc(staging_bytes);
	if (!staging) {
		fprintf(stderr, "Error: malloc failed for %lu bytes of staging while loading %s...\n", (unsigned long) staging_bytes, filename);
		fclose(file);
		return -1;
	}
	int ret = 0;
#define UPLOAD(dev, host, bytes) do { \
		if (!ret && ((handle->submit_inbound_transfer)(handle, stream_id, (dev), (host), (bytes)) || (handle->sync_stream)(handle, stream_id))) { \
			fprintf(stderr, "Error: failed to transfer weights of %s to the device...\n", filename); \
			ret = -1; \
		} \
	} while (0)
	if (ffn_norm_weight) {
		ret = read_at(file, filename, off.w_ffn_norm, staging, D * el);
		UPLOAD(ffn_norm_weight, staging, D * el);
	}
	if (!ret) {
		ret = read_at(file, filename, off.w_router, staging, router);
		UPLOAD(layer->w_router, staging, router);
	}
	for (uint64_t e = 0; e < E && !ret; e++) {
		const uint64_t base = e * off.expert_stride;
		ret = read_at(file, filename, off.w_1 + base, staging, up);
		if (!ret) {
			ret = read_at(file, filename, off.w_3 + base, staging + up, up);
		}
		if (!ret) {
			ret = read_at(file, filename, off.w_2 + base, staging + 2 * up, up);
		}
		UPLOAD((uint8_t *) layer->w1 + e * layer->expert_stride_bytes, staging, up);
		UPLOAD((uint8_t *) layer->w3 + e * layer->expert_stride_bytes, staging + up, up);
		UPLOAD((uint8_t *) layer->w2 + e * layer->expert_stride_bytes, staging + 2 * up, up);
	}
#undef UPLOAD
	free(staging);
	fclose(file);
	return ret;
}

/* the reference's naming (dataflow_transformer.c:77-134): seq_id == -1 marks model weights (is_bwd: their gradients),
 * layer_id -2 is the embedding, -1 the head, >= 0 a block */
int amd_moe_saved_array_path(char * path, size_t path_bytes, const char * save_dir, int layer_id, int seq_id, int chunk_id,
							 int is_bwd, const char * name) {
	if (!path || !save_dir || !name || layer_id < -2) {
		fprintf(stderr, "Error: invalid layer id (should be -2 (embedding), -1 (head), or layer id >= 0)): %d\n", layer_id);
		return -1;
	}
	int n;
	if (seq_id == -1) {
		const char * root = is_bwd ? "model_grads" : "model";
		if (layer_id >= 0) {
			n = snprintf(path, path_bytes, "%s/%s/layers/%d/%s.dat", save_dir, root, layer_id, name);
		} else {
			n = snprintf(path, path_bytes, "%s/%s/%s/%s.dat", save_dir, root, layer_id == -2 ? "embedding" : "head", name);
		}
	} else if (layer_id >= 0) {
		n = snprintf(path, path_bytes, "%s/%s/%d/seq_%d_chunk_%d_%s.dat", save_dir, is_bwd ? "layers_bwd" : "layers_fwd", layer_id, seq_id, chunk_id, name);
	} else {
		const char * where = layer_id == -2 ? (is_bwd ? "embedding_bwd" : "embedding_fwd") : (is_bwd ? "head_bwd" : "head_fwd");
		n = snprintf(path, path_bytes, "%s/%s/seq_%d_chunk_%d_%s.dat", save_dir, where, seq_id, chunk_id, name);
	}
	if (n < 0 || (size_t) n >= path_bytes) {
		fprintf(stderr, "Error: path of saved array %s does not fit %zu bytes...\n", name, path_bytes);
		return -1;
	}
	return 0;
}

int amd_moe_save_array(Dataflow_Handle * handle, int stream_id, const char * save_dir, int layer_id, int seq_id, int chunk_id,
					   int is_bwd, const char * name, void * dev_ptr, int M, int N, DataflowDatatype dt) {
	char path[1024];
	if (!handle || M < 0 || N < 0 || amd_moe_saved_array_path(path, sizeof(path), save_dir, layer_id, seq_id, chunk_id, is_bwd, name)) {
		return -1;
	}
	size_t num_els = (size_t) M * (size_t) N;
	size_t el_size = dataflow_sizeof_element(dt);
	if (el_size == 0) {
		fprintf(stderr, "Error: cannot save %s with element type %s...\n", name, dataflow_datatype_as_string(dt));
		return -1;
	}
	void * host = malloc(num_els * el_size + 1);
	if (!host) {
		fprintf(stderr, "Error: malloc failed while saving %s...\n", name);
		return -1;
	}
	if (num_els > 0 && ((handle->submit_outbound_transfer)(handle, stream_id, host, dev_ptr, num_els * el_size) || (handle->sync_stream)(handle, stream_id))) {
		fprintf(stderr, "Error: failed to copy %s back from the device...\n", name);
		free(host);
		return -1;
	}
	/* the directory has to exist, as for the reference */
	FILE * fp = fopen(path, "wb");
	if (!fp) {
		fprintf(stderr, "Error: failed to save %s, because couldn't open file: %s...\n", name, path);
		free(host);
		return -1;
	}
	size_t written = fwrite(host, el_size, num_els, fp);
	free(host);
	if (fclose(fp) != 0 || written != num_els) {
		fprintf(stderr, "Error: failed to write to file %s, wrote %zu elements instead of %zu\n", path, written, num_els);
		return -1;
	}
	return 0;
}
