/*
 * dataflow_core.c -- the few libdataflow services the MoE backend needs: dtype sizes/strings,
 * scalar bf16 conversion, SHA-256 fingerprints of op skeletons and the open-addressing op table.
 *
 * Same contracts as libdataflow/src/dataflow_datatype/dataflow_datatype.c:4-79,
 * libdataflow/src/dataflow_fingerprint/dataflow_fingerprint.c:77-85 (SHA-256 of the bytes handed in) and
 * libdataflow/src/dataflow_table/dataflow_table.c (memcpy keys/values, linear probing, 1-bits mark empty
 * slots), written from scratch and without OpenSSL so the backend has no dependency besides HIP.
 */
#include "dataflow_amd.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ datatypes */

size_t dataflow_sizeof_element(DataflowDatatype arr_dtype) {
	switch (arr_dtype) {
		case DATAFLOW_FP64: case DATAFLOW_UINT64: return 8;
		case DATAFLOW_FP32: case DATAFLOW_UINT32: return 4;
		case DATAFLOW_FP16: case DATAFLOW_BF16: case DATAFLOW_UINT16: return 2;
		case DATAFLOW_FP8E4M3: case DATAFLOW_FP8E5M2: case DATAFLOW_UINT8: return 1;
		case DATAFLOW_LONG: return sizeof(long);
		case DATAFLOW_INT: return sizeof(int);
		default: return 0;
	}
}

/* Upper-case names; these strings are part of every op nickname and therefore of every fingerprint. */
char * dataflow_datatype_as_string(DataflowDatatype dtype) {
	static char * const names[] = {
		[DATAFLOW_VOID] = "VOID", [DATAFLOW_FP64] = "FP64", [DATAFLOW_FP32] = "FP32", [DATAFLOW_FP16] = "FP16",
		[DATAFLOW_BF16] = "BF16", [DATAFLOW_FP8E4M3] = "FP8E4M3", [DATAFLOW_FP8E5M2] = "FP8E5M2",
		[DATAFLOW_UINT64] = "UINT64", [DATAFLOW_UINT32] = "UINT32", [DATAFLOW_UINT16] = "UINT16",
		[DATAFLOW_UINT8] = "UINT8", [DATAFLOW_LONG] = "LONG", [DATAFLOW_INT] = "INT",
	};
	if ((int) dtype >= (int) DATAFLOW_VOID && (int) dtype <= (int) DATAFLOW_INT) {
		return names[dtype];
	}
	return "UNKNOWN";
}

float solo_bf16_to_fp32(uint16_t a) {
	uint32_t bits = ((uint32_t) a) << 16;
	float f;
	memcpy(&f, &bits, sizeof(f));
	return f;
}

uint16_t solo_fp32_to_bf16(float f) {
	uint32_t bits;
	memcpy(&bits, &f, sizeof(bits));
	if ((bits & 0x7fffffffu) > 0x7f800000u) {
		return (uint16_t) ((bits >> 16) | 0x0040u);
	}
	bits += 0x7fffu + ((bits >> 16) & 1u);
	return (uint16_t) (bits >> 16);
}

/* ------------------------------------------------------------------ SHA-256 (FIPS 180-4) */

static const uint32_t sha256_k[64] = {
	0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5,
	0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
	0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
	0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
	0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
	0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
	0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3,
	0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2
};

static inline uint32_t rotr32(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

static void sha256_block(uint32_t state[8], const uint8_t block[64]) {
	uint32_t w[64];
	for (int i = 0; i < 16; i++) {
		w[i] = ((uint32_t) block[4 * i] << 24) | ((uint32_t) block[4 * i + 1] << 16) | ((uint32_t) block[4 * i + 2] << 8) | (uint32_t) block[4 * i + 3];
	}
	for (int i = 16; i < 64; i++) {
		uint32_t s0 = rotr32(w[i - 15], 7) ^ rotr32(w[i - 15], 18) ^ (w[i - 15] >> 3);
		uint32_t s1 = rotr32(w[i - 2], 17) ^ rotr32(w[i - 2], 19) ^ (w[i - 2] >> 10);
		w[i] = w[i - 16] + s0 + w[i - 7] + s1;
	}
	uint32_t a = state[0], b = state[1], c = state[2], d = state[3], e = state[4], f = state[5], g = state[6], h = state[7];
	for (int i = 0; i < 64; i++) {
		uint32_t S1 = rotr32(e, 6) ^ rotr32(e, 11) ^ rotr32(e, 25);
		uint32_t ch = (e & f) ^ (~e & g);
		uint32_t t1 = h + S1 + ch + sha256_k[i] + w[i];
		uint32_t S0 = rotr32(a, 2) ^ rotr32(a, 13) ^ rotr32(a, 22);
		uint32_t mj = (a & b) ^ (a & c) ^ (b & c);
		uint32_t t2 = S0 + mj;
		h = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
	}
	state[0] += a; state[1] += b; state[2] += c; state[3] += d; state[4] += e; state[5] += f; state[6] += g; state[7] += h;
}

int dataflow_do_fingerprinting(void * data, uint64_t num_bytes, uint8_t * ret_fingerprint) {
	if (!data || !ret_fingerprint) {
		fprintf(stderr, "Error: fingerprinting needs a data pointer and a 32-byte destination...\n");
		return -1;
	}
	uint32_t state[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
	const uint8_t * p = (const uint8_t *) data;
	uint64_t full = num_bytes / 64;
	for (uint64_t i = 0; i < full; i++) {
		sha256_block(state, p + 64 * i);
	}
	uint8_t tail[128];
	uint64_t rem = num_bytes - 64 * full;
	memset(tail, 0, sizeof(tail));
	memcpy(tail, p + 64 * full, rem);
	tail[rem] = 0x80;
	int tail_blocks = (rem + 1 + 8 <= 64) ? 1 : 2;
	uint64_t bit_len = num_bytes * 8;
	for (int i = 0; i < 8; i++) {
		tail[64 * tail_blocks - 1 - i] = (uint8_t) (bit_len >> (8 * i));
	}
	for (int i = 0; i < tail_blocks; i++) {
		sha256_block(state, tail + 64 * i);
	}
	for (int i = 0; i < 8; i++) {
		ret_fingerprint[4 * i] = (uint8_t) (state[i] >> 24);
		ret_fingerprint[4 * i + 1] = (uint8_t) (state[i] >> 16);
		ret_fingerprint[4 * i + 2] = (uint8_t) (state[i] >> 8);
		ret_fingerprint[4 * i + 3] = (uint8_t) state[i];
	}
	return 0;
}

/* ------------------------------------------------------------------ op table */

/* Slot i is the byte range [i*(key+value), (i+1)*(key+value)) of items; bit (i & 63) of
 * is_empty_bit_vector[i >> 6] is 1 while the slot is free. Single-threaded by contract. */

static inline uint64_t slot_bytes(const Dataflow_Table * t) { return t->config.key_size_bytes + t->config.value_size_bytes; }
static inline int slot_is_empty(const Dataflow_Table * t, uint64_t i) { return (int) ((t->is_empty_bit_vector[i >> 6] >> (i & 63)) & 1ULL); }
static inline void slot_mark(Dataflow_Table * t, uint64_t i, int empty) {
	if (empty) { t->is_empty_bit_vector[i >> 6] |= (1ULL << (i & 63)); }
	else { t->is_empty_bit_vector[i >> 6] &= ~(1ULL << (i & 63)); }
}

static int table_alloc(Dataflow_Table * table, uint64_t size) {
	uint64_t words = (size + 63) / 64;
	table->is_empty_bit_vector = (uint64_t *) malloc(words * sizeof(uint64_t));
	table->items = calloc(size, slot_bytes(table));
	if (!table->is_empty_bit_vector || !table->items) {
		free(table->is_empty_bit_vector);
		free(table->items);
		table->is_empty_bit_vector = NULL;
		table->items = NULL;
		return -1;
	}
	for (uint64_t w = 0; w < words; w++) {
		uint64_t lo = 64 * w;
		table->is_empty_bit_vector[w] = (size - lo >= 64) ? ~0ULL : ((1ULL << (size - lo)) - 1ULL);
	}
	table->size = size;
	return 0;
}

int dataflow_init_table(Dataflow_Table * table, Hash_Func hash_func, uint64_t key_size_bytes, uint64_t value_size_bytes,
						uint64_t min_table_size, uint64_t max_table_size, float load_factor, float shrink_factor) {
	if (!table || !hash_func || key_size_bytes == 0 || min_table_size == 0 || max_table_size < min_table_size) {
		fprintf(stderr, "Error: bad arguments to dataflow_init_table...\n");
		return -1;
	}
	table->config.hash_func = hash_func;
	table->config.key_size_bytes = key_size_bytes;
	table->config.value_size_bytes = value_size_bytes;
	table->config.min_size = min_table_size;
	table->config.max_size = max_table_size;
	table->config.load_factor = load_factor;
	table->config.shrink_factor = shrink_factor;
	table->cnt = 0;
	if (table_alloc(table, min_table_size)) {
		fprintf(stderr, "Error: could not allocate op table of %lu slots...\n", (unsigned long) min_table_size);
		return -1;
	}
	return 0;
}

void dataflow_destroy_table(Dataflow_Table * table) {
	if (!table) {
		return;
	}
	free(table->is_empty_bit_vector);
	free(table->items);
	table->is_empty_bit_vector = NULL;
	table->items = NULL;
	table->cnt = 0;
	table->size = 0;
}

/* place (key,value) into the first free slot at or after hash(key); caller guarantees a free slot exists */
static void table_place(Dataflow_Table * table, const void * key, const void * value) {
	uint64_t sb = slot_bytes(table);
	uint64_t i = table->config.hash_func((void *) key, table->size);
	while (!slot_is_empty(table, i)) {
		i = (i + 1 == table->size) ? 0 : i + 1;
	}
	uint8_t * dst = (uint8_t *) table->items + i * sb;
	memcpy(dst, key, table->config.key_size_bytes);
	if (table->config.value_size_bytes) {
		memcpy(dst + table->config.key_size_bytes, value, table->config.value_size_bytes);
	}
	slot_mark(table, i, 0);
}

static int table_resize(Dataflow_Table * table, uint64_t new_size) {
	Dataflow_Table old = *table;
	if (table_alloc(table, new_size)) {
		*table = old;
		return -1;
	}
	uint64_t sb = slot_bytes(&old);
	for (uint64_t i = 0; i < old.size; i++) {
		if (!slot_is_empty(&old, i)) {
			const uint8_t * src = (const uint8_t *) old.items + i * sb;
			table_place(table, src, src + old.config.key_size_bytes);
		}
	}
	free(old.is_empty_bit_vector);
	free(old.items);
	return 0;
}

long dataflow_find_table(Dataflow_Table * table, void * key, bool to_copy_value, void ** ret_value) {
	if (ret_value && !to_copy_value) {
		*ret_value = NULL;
	}
	if (!table || !table->items || table->size == 0) {
		return -1;
	}
	uint64_t sb = slot_bytes(table);
	uint64_t i = table->config.hash_func(key, table->size);
	for (uint64_t probes = 0; probes < table->size; probes++) {
		if (slot_is_empty(table, i)) {
			break;
		}
		uint8_t * slot = (uint8_t *) table->items + i * sb;
		if (memcmp(slot, key, table->config.key_size_bytes) == 0) {
			if (ret_value) {
				if (to_copy_value) {
					memcpy(*ret_value, slot + table->config.key_size_bytes, table->config.value_size_bytes);
				} else {
					*ret_value = slot + table->config.key_size_bytes;
				}
			}
			return (long) i;
		}
		i = (i + 1 == table->size) ? 0 : i + 1;
	}
	if (ret_value && to_copy_value) {
		*ret_value = NULL;
	}
	return -1;
}

int dataflow_insert_table(Dataflow_Table * table, void * key, void * value) {
	if (!table || !table->items) {
		return -1;
	}
	if (dataflow_find_table(table, key, false, NULL) >= 0) {
		fprintf(stderr, "Error: key already present in table...\n");
		return -1;
	}
	if (table->size < table->config.max_size && (float) (table->cnt + 1) > (float) table->size * table->config.load_factor && table->config.load_factor > 0.0f) {
		uint64_t grown = (uint64_t) ((float) table->size / table->config.load_factor);
		if (grown <= table->size) { grown = table->size * 2; }
		if (grown > table->config.max_size) { grown = table->config.max_size; }
		if (table_resize(table, grown)) {
			fprintf(stderr, "Error: could not grow table to %lu slots...\n", (unsigned long) grown);
			return -1;
		}
	}
	if (table->cnt >= table->size) {
		fprintf(stderr, "Error: table is full (%lu slots)...\n", (unsigned long) table->size);
		return -1;
	}
	table_place(table, key, value);
	table->cnt++;
	return 0;
}

int dataflow_remove_table(Dataflow_Table * table, void * key, void * ret_value) {
	long at = dataflow_find_table(table, key, false, NULL);
	if (at < 0) {
		return -1;
	}
	uint64_t sb = slot_bytes(table);
	uint64_t i = (uint64_t) at;
	if (ret_value) {
		memcpy(ret_value, (uint8_t *) table->items + i * sb + table->config.key_size_bytes, table->config.value_size_bytes);
	}
	/* backward-shift deletion keeps every remaining key reachable from its home slot */
	uint64_t hole = i;
	uint64_t j = (hole + 1 == table->size) ? 0 : hole + 1;
	while (!slot_is_empty(table, j)) {
		uint8_t * cand = (uint8_t *) table->items + j * sb;
		uint64_t home = table->config.hash_func(cand, table->size);
		/* cand may move into the hole if its home is not in the cyclic interval (hole, j] */
		int between = (hole < j) ? (home > hole && home <= j) : (home > hole || home <= j);
		if (!between) {
			memcpy((uint8_t *) table->items + hole * sb, cand, sb);
			hole = j;
		}
		j = (j + 1 == table->size) ? 0 : j + 1;
	}
	memset((uint8_t *) table->items + hole * sb, 0, sb);
	slot_mark(table, hole, 1);
	table->cnt--;
	return 0;
}
