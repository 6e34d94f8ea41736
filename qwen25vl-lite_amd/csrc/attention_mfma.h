// Entry points of the matrix-core attention library that callers outside this package may use
// directly (the library is compiled per head size, -DHD=...; every function returns 0 or one of
// the QVL_ERR_* codes of common.h).
#pragma once
#include <hip/hip_runtime.h>

// Floats in the library's own array for partial results: 8 MiB, held on every GPU the library
// runs on until the process ends.  The library is compiled once per head size (and once more for
// its wide kind): every such variant that a process loads carries an array of its own, so a
// process that uses n head sizes holds n times 8 MiB per GPU.
#define QVL_ATTN_STATIC_SCRATCH_FLOATS (2 * 1024 * 1024)

extern "C" {

// Floats of partial results a call with these sizes produces (nsplit > 1 only).
long long qvl_attn_mfma_scratch_floats(int num_tiles, int nkv, int nsplit);

// Attention of few column tiles (decode): the waves of a block share a tile; with nsplit > 1 the
// keys of a tile are cut into nsplit ranges of keys_per_split keys (a multiple of 32) whose partial
// results go through `scratch` (qvl_attn_mfma_scratch_floats() floats, the caller's) and are
// merged by a second kernel.  tile_req and tile_ct may both be null: tile i is then the one tile of
// request i; cu_q may be null: every request then brings one token, request r the token r (a step
// of decoded tokens only: the kernel starts without reading either).
int qvl_attn_mfma_coop(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                       const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                       int num_tiles, void* out, void* scratch, int nq, int nkv, int ps, int window, float scale,
                       int nsplit, int keys_per_split, hipStream_t stream);

// The same call for callers that cannot allocate device memory: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.
// The partial results go through an array inside the library (QVL_ATTN_STATIC_SCRATCH_FLOATS
// floats per GPU); the call allocates and frees nothing.  Inputs and outputs are the caller's, as
// above.  A call whose partial results would not fit (qvl_attn_mfma_scratch_floats(...) beyond
// qvl_attn_mfma_static_scratch_floats()) is refused with QVL_ERR_LIMIT (4) and launches nothing.
// All calls on one GPU share that GPU's array: calls that may overlap there (different streams,
// different threads) race; calls on one stream do not.  The array keeps the last call's contents;
// no call depends on them.  The device current at the call must be the one `stream` belongs to.
// The array's address on a device is looked up at the first call there, or by
// qvl_attn_mfma_coop_static_init() with that device current (a caller that captures a graph makes
// that call, or one uncaptured call, beforehand).
int qvl_attn_mfma_coop_static(const void* q, const void* kc, const void* vc, const void* bt, int table_width,
                              const void* cu_q, const void* ctx_len, const void* tile_req, const void* tile_ct,
                              int num_tiles, void* out, int nq, int nkv, int ps, int window, float scale,
                              int nsplit, int keys_per_split, hipStream_t stream);
int qvl_attn_mfma_coop_static_init();
long long qvl_attn_mfma_static_scratch_floats();

}  // extern "C"
