// Entry points of attention over the paged cache.
//
// qe_attention          any sizes, float32 or bfloat16, one wave per (token, head); for all
//                       tokens of the batch or for a list of them
// qe_attention_decode_* bfloat16 MFMA kernel for tokens that are the single new token of their
//                       request (see attention_decode.hip)
// qe_attention_prefill_run  bfloat16 MFMA kernel for portions of prompts (see attention_prefill.hip)
#include "common.h"

int qe_attention_generic(const void* q, void* out, const void* cache, const int* positions,
                         const int* tok_seq, const int* block_table, int max_blocks, const int* tokens,
                         int T, int Hq, int Hkv, int D, int P, float scale, int window, int dt_a,
                         hipStream_t stream);
bool qe_attention_decode_ok(int Hq, int Hkv, int D, int P, int dt_a);
size_t qe_attention_decode_workspace(int n_dec, int Hq, int D, int num_splits);
int qe_attention_decode(const void* q, void* out, const void* cache, const int* dec_tokens, int n_dec,
                        const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                        const int* shared_keys, int Hq, int Hkv, int D, int P, float scale, int window, int max_position,
                        int split_keys, void* workspace, size_t workspace_bytes, hipStream_t stream);

int qe_attention_prefill(const void* q, void* out, const void* cache, const int* tiles, int num_tiles,
                         const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                         int Hq, int Hkv, int D, int P, float scale, int window, int groups,
                         int seg_keys, int max_keys, int keys_row, void* workspace, size_t workspace_bytes,
                         hipStream_t stream);
int qe_attention_prefill_segment_keys(long blocks, int max_keys);
int qe_attention_prefill_segments(long blocks);
int qe_attention_prefill_uncut_keys();
size_t qe_attention_prefill_workspace(int num_tiles, int Hq, int Hkv, int D, int segments);

int qe_attention_prefill_tile_rows(int Hq, int Hkv);
int qe_attention_prefill_tiles(const int* portions, int n_portions, int rows_per_tile, int* tiles, int max_groups,
                               hipStream_t stream);

// The tile list for qe_attention_prefill_run from portions [n_portions][2] = (first row, rows) that lie
// on the device: tiles [4 max_groups][2], whatever is beyond the portions' groups being groups of no
// rows.  The caller guarantees that the portions have at most max_groups groups of 4 tiles.
extern "C" int qe_attention_prefill_tiles_run(const int* portions, int n_portions, int rows_per_tile, int* tiles,
                                              int max_groups, hipStream_t stream) {
    return qe_attention_prefill_tiles(portions, n_portions, rows_per_tile, tiles, max_groups, stream);
}

// rows of a tile for these head counts
extern "C" int qe_attention_prefill_rows(int Hq, int Hkv) {
    if (Hq <= 0 || Hkv <= 0 || Hq % Hkv) return 0;
    return qe_attention_prefill_tile_rows(Hq, Hkv);
}

// Into segments of how many keys the prefill kernel's walks are best cut for num_tiles tiles whose
// rows see at most max_keys keys: 0 for not at all.
extern "C" int qe_attention_prefill_plan(int num_tiles, int Hq, int Hkv, int max_keys) {
    if (num_tiles <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || max_keys <= 0) return 0;
    const int R = qe_attention_prefill_tile_rows(Hq, Hkv);
    return qe_attention_prefill_segment_keys((long)(num_tiles / 4) * Hkv * ((Hq / Hkv) / (32 / R)), max_keys);
}

// Into how many segments at most (1: not at all): for a caller that leaves their length to the device.
extern "C" int qe_attention_prefill_plan_segments(int num_tiles, int Hq, int Hkv) {
    if (num_tiles <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv) return 1;
    const int R = qe_attention_prefill_tile_rows(Hq, Hkv);
    return qe_attention_prefill_segments((long)(num_tiles / 4) * Hkv * ((Hq / Hkv) / (32 / R)));
}

// up to this many keys the plan is never to cut
extern "C" int qe_attention_prefill_plan_uncut_keys() { return qe_attention_prefill_uncut_keys(); }

// bytes of workspace for segments of seg_keys keys (> 0)
extern "C" long qe_attention_prefill_workspace_bytes(int num_tiles, int Hq, int Hkv, int D, int max_keys, int seg_keys) {
    if (seg_keys <= 0 || max_keys <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv) return 0;
    return (long)qe_attention_prefill_workspace(num_tiles, Hq, Hkv, D, (max_keys + seg_keys - 1) / seg_keys);
}

// ... and for a number of segments
extern "C" long qe_attention_prefill_workspace_bytes_for(int num_tiles, int Hq, int Hkv, int D, int segments) {
    if (segments <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv) return 0;
    return (long)qe_attention_prefill_workspace(num_tiles, Hq, Hkv, D, segments);
}

// tiles: num_tiles pairs (first row of q, rows <= qe_attention_prefill_rows) of consecutive new
// tokens of one request.  Takes what qe_attention_prefill_supported takes.  groups: wave groups
// a block that share the key tiles between them, 1 or 2, or 0 to choose by the number of blocks.
// seg_keys: 0, or the keys of a segment (a multiple of 64) into which the walks are cut; then no row
// sees more than max_keys keys and the workspace has qe_attention_prefill_workspace_bytes bytes.  Or
// minus a number of segments (2 to 8): the kernels take the keys that row keys_row of q sees (no row
// sees more) from its position and cut them into that many segments, or fewer, themselves; the
// workspace then has qe_attention_prefill_workspace_bytes_for that number.
extern "C" int qe_attention_prefill_run(const void* q, void* out, const void* cache, const int* tiles,
                                        int num_tiles, const int* positions, const int* tok_seq,
                                        const int* block_table, int max_blocks, int Hq, int Hkv, int D, int P,
                                        float scale, int window, int groups, int seg_keys, int max_keys,
                                        int keys_row, void* workspace, long workspace_bytes, hipStream_t stream) {
    QE_REQUIRE(num_tiles >= 0 && Hq > 0 && Hkv > 0 && max_blocks > 0 && window >= 0 && workspace_bytes >= 0,
               "prefill attention: bad sizes");
    return qe_attention_prefill(q, out, cache, tiles, num_tiles, positions, tok_seq, block_table, max_blocks,
                                Hq, Hkv, D, P, scale, window, groups, seg_keys, max_keys, keys_row, workspace,
                                (size_t)workspace_bytes, stream);
}

// tokens: null for all T rows of q, else n_tokens row indices.
extern "C" int qe_attention(const void* q, void* out, const void* cache, const int* positions,
                            const int* tok_seq, const int* block_table, int max_blocks, const int* tokens,
                            int n_tokens, int Hq, int Hkv, int D, int P, float scale, int window, int dt_a,
                            hipStream_t stream) {
    QE_REQUIRE(n_tokens >= 0 && Hq > 0 && Hkv > 0 && D > 0 && P > 0 && max_blocks > 0, "attention: bad sizes");
    QE_REQUIRE(Hq % Hkv == 0, "attention: %d query heads are no multiple of %d key/value heads", Hq, Hkv);
    QE_REQUIRE(window >= 0, "attention: negative window");
    if (n_tokens == 0) return 0;
    return qe_attention_generic(q, out, cache, positions, tok_seq, block_table, max_blocks, tokens, n_tokens,
                                Hq, Hkv, D, P, scale, window, dt_a, stream);
}

extern "C" int qe_attention_decode_supported(int Hq, int Hkv, int D, int P, int dt_a) {
    return qe_attention_decode_ok(Hq, Hkv, D, P, dt_a) ? 1 : 0;
}

extern "C" int qe_attention_prefill_supported(int Hq, int Hkv, int D, int P, int dt_a) {
    return (qe_attention_decode_ok(Hq, Hkv, D, P, dt_a) && (P & (P - 1)) == 0) ? 1 : 0;
}

extern "C" long qe_attention_decode_workspace_bytes(int n_dec, int Hq, int D, int max_position, int split_keys) {
    return (long)qe_attention_decode_workspace(n_dec, Hq, D, max_position / split_keys + 1);
}

int qe_attention_decode_fused(const void* qkv, void* out, void* cache, const int* dec_tokens, int n_dec,
                              const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                              const int* shared_keys, const int* slots, const float* q_w, const float* k_w, float eps,
                              const float* table, int Hq, int Hkv, int D, int P, float scale, int window, int max_position,
                              int split_keys, void* workspace, size_t workspace_bytes, hipStream_t stream);

// Decode attention with the q/k norm, the rotation and the cache write of the new tokens inside:
// qkv [T, (Hq + 2 Hkv) D] bfloat16 as the projection left it; q_w, k_w [D] float or null; table
// [positions, D] float rows [cos | sin] (a rotation over the whole head) or null; slots [T]: where
// each row's own key and value go in the cache (negative: nowhere).  shared_keys: null, or per row of the
// block table how many of the request's first keys other requests read too (a hint for the caches: those
// keys are left in them, the others stream past).  Takes what qe_attention_decode_supported takes.
extern "C" int qe_attention_decode_fused_run(const void* qkv, void* out, void* cache, const int* dec_tokens,
                                             int n_dec, const int* positions, const int* tok_seq,
                                             const int* block_table, int max_blocks, const int* shared_keys,
                                             const int* slots,
                                             const float* q_w, const float* k_w, float eps, const float* table,
                                             int Hq, int Hkv, int D, int P, float scale, int window,
                                             int max_position, int split_keys, void* workspace,
                                             long workspace_bytes, hipStream_t stream) {
    QE_REQUIRE(Hq > 0 && Hkv > 0 && max_blocks > 0 && window >= 0 && max_position >= 0, "decode attention: bad sizes");
    return qe_attention_decode_fused(qkv, out, cache, dec_tokens, n_dec, positions, tok_seq, block_table,
                                     max_blocks, shared_keys, slots, q_w, k_w, eps, table, Hq, Hkv, D, P, scale, window,
                                     max_position, split_keys, workspace, (size_t)workspace_bytes, stream);
}

extern "C" int qe_attention_decode_run(const void* q, void* out, const void* cache, const int* dec_tokens,
                                       int n_dec, const int* positions, const int* tok_seq,
                                       const int* block_table, int max_blocks, const int* shared_keys,
                                       int Hq, int Hkv, int D, int P, float scale, int window,
                                       int max_position, int split_keys, void* workspace, long workspace_bytes,
                                       hipStream_t stream) {
    QE_REQUIRE(Hq > 0 && Hkv > 0 && max_blocks > 0 && window >= 0 && max_position >= 0, "decode attention: bad sizes");
    return qe_attention_decode(q, out, cache, dec_tokens, n_dec, positions, tok_seq, block_table, max_blocks,
                               shared_keys, Hq, Hkv, D, P, scale, window, max_position, split_keys, workspace,
                               (size_t)workspace_bytes, stream);
}
