/* Host-side helpers of the KV path with a C ABI: the fixed-shape step descriptors a captured
 * (HIP graph) decode step reads.  They restate crates/warp34-host/src/model/graph_io.rs
 * (decode_graph_bucket :585-595, BatchedDecodeGraphIo::pack_meta :789-871 and the pointer
 * accessors :746-787); the reference keeps them in Rust, so none of these symbols has a
 * counterpart in its C header.  Pure host code: callable without a GPU. */
#ifndef WARP34_HOST_H
#define WARP34_HOST_H

#include <stddef.h>
#include <stdint.h>

#include "warp34_kv.h"

#ifdef __cplusplus
extern "C" {
#endif

#define WARP34_HOST_MAX_BATCHED_DECODE_REQS 16
/* bytes of one batched-decode blob: 177 i32 words, padding to 64 bytes, 48 mask bytes */
#define WARP34_HOST_DECODE_BLOB_BYTES 816

/* Rows of the captured graph that serves num_reqs one-token requests (1, 2, 4, 8, 16); 0: none. */
int warp34_host_decode_graph_bucket(int num_reqs);

/* Packs the blob of a batched one-token decode step.  Request r has token tokens[r], context
 * length ctx_lens_before[r] and the block table block_tables[r * bt_stride .. + block_table_lens[r]).
 * Rows behind num_reqs are padding: masked out, write slot -1.  Returns 0, or 1 for an invalid
 * batch (no / too many requests, a table too short for position ctx_lens_before[r]). */
int warp34_host_pack_batched_decode_blob(const int32_t* tokens, const int32_t* ctx_lens_before,
                                         const int32_t* block_tables, const int32_t* block_table_lens,
                                         int bt_stride, int num_reqs, int page_size, uint8_t* blob_out);

/* The attention descriptor of a replay with `bucket` rows over a blob at device address dev_blob
 * and block tables [16][max_blocks_per_req] at dev_block_tables. */
void warp34_host_batched_decode_batch_at(uint64_t dev_blob, uint64_t dev_block_tables, int bucket,
                                         int max_blocks_per_req, int max_seq_len, int mask_mode, float sm_scale,
                                         warp34_attention_batch* out);

#ifdef __cplusplus
}
#endif
#endif
