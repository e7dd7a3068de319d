// The C entry points of the attention library (attention.hip).  Every call launches on `stream`
// and returns 0, a negative DN_ERR_* code (nothing was launched) or a positive hipError_t.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// the scratch of dn_attention_decode_static cannot hold what the call needs
#define DN_ERR_SCRATCH (-3)

// Floats of split results that dn_attention_decode_static can hold per GPU (1 MiB):
// n_tiles * H * n_splits * (dh + 2) must not exceed it.
#define DN_DECODE_STATIC_SCRATCH_FLOATS (256 * 1024)

extern "C" {

// All kernels: q [T, ldq], out [T, ldo] (ldo == 0: packed rows), k_pool [n_pages, Hkv, page_size, dh],
// v_pool [n_pages, Hkv, dh, page_size], block_tables int32 [S, max_blocks], tile tables int32 [n_tiles].

// any dtype (DN_F32, DN_BF16), any head size that is a multiple of 16 up to 256: tiles of up to 16 rows
int dn_attention(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                 const int32_t* block_tables, int max_blocks, const int32_t* tile_seq, const int32_t* tile_row0,
                 const int32_t* tile_nrows, const int32_t* tile_pos0, int n_tiles, int H, int Hkv, int dh,
                 int page_size, float scale, int window, int dtype, hipStream_t stream);

// the same kernels' arithmetic for a step of single rows (tile s = request s = row s), every tile of keys a
// workgroup of its own; part: n_tiles * H * ceil(max_context / dn_attention_rows_tile(dh)) * (dh + 2) floats
int dn_attention_rows_tile(int dh);
int dn_attention_rows(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                      const int32_t* block_tables, int max_blocks, const int32_t* tile_seq, const int32_t* tile_pos0,
                      int n_tiles, float* part, int max_context, int H, int Hkv, int dh, int page_size, float scale,
                      int window, int dtype, hipStream_t stream);

// bfloat16, matrix cores: tiles of up to 128 rows
int dn_attention_flash(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                       const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                       const int32_t* tile_row0, const int32_t* tile_nrows, const int32_t* tile_pos0, int n_tiles,
                       int H, int Hkv, int dh, int page_size, float scale, int window, hipStream_t stream);

// bfloat16, one row per request (tile s = request s = row s); the context is cut into n_splits runs of
// `chunks` chunks of waves * 64 keys; part: device memory for n_tiles * H * n_splits * (dh + 2) floats
// of split results (not touched when n_splits == 1).  tile_row0 is not read: tile s is row s of q and
// of out and row s of the block tables, whatever the table says (the kernels address them by the
// workgroup's index, so that these loads do not wait for the table's); a caller whose tile s is
// another row takes dn_attention_flash or dn_attention.
int dn_attention_decode(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                        const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                        const int32_t* tile_row0, const int32_t* tile_pos0, int n_tiles, float* part, int n_splits,
                        int chunks, int waves, int H, int Hkv, int dh, int page_size, float scale, int window,
                        hipStream_t stream);

// dn_attention_decode for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
// The split results go to an array that the library itself holds on every GPU it runs on
// (DN_DECODE_STATIC_SCRATCH_FLOATS floats, until the process ends) in place of `part`; the call
// allocates and frees nothing.  The same kernels, the same results bit for bit.
//  * n_tiles * H * n_splits * (dh + 2) > DN_DECODE_STATIC_SCRATCH_FLOATS (and n_splits > 1):
//    DN_ERR_SCRATCH, nothing is launched.
//  * Every call on a GPU shares that GPU's array, which keeps the last call's contents.  Nothing in
//    it has to start at zero: the first kernel writes every entry that the second reads.  Two calls
//    that overlap in time on one GPU (different streams, different threads) race on it: callers
//    order them on one stream.
//  * The array's address is looked up once per GPU, at the first call with that GPU current.
int dn_attention_decode_static(const void* q, int ldq, void* out, int ldo, const void* k_pool, const void* v_pool,
                               const int32_t* block_tables, int max_blocks, const int32_t* tile_seq,
                               const int32_t* tile_row0, const int32_t* tile_pos0, int n_tiles, int n_splits,
                               int chunks, int waves, int H, int Hkv, int dh, int page_size, float scale,
                               int window, hipStream_t stream);
}
