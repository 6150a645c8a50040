// Entry point of attention over the paged cache: picks a kernel for the shape.
#include "common.h"

int qe_attention_generic(const void* q, void* out, const void* cache, const int* positions,
                         const int* tok_seq, const int* block_table, int max_blocks, int T, int Hq,
                         int Hkv, int D, int P, float scale, int window, int dt_a, hipStream_t stream);

// algo: 0 = choose, 1 = generic 32-bit kernel.
extern "C" int qe_attention(const void* q, void* out, const void* cache, const int* positions,
                            const int* tok_seq, const int* block_table, int max_blocks, int T,
                            int Hq, int Hkv, int D, int P, float scale, int window, int dt_a, int algo,
                            hipStream_t stream) {
    QE_REQUIRE(T >= 0 && Hq > 0 && Hkv > 0 && D > 0 && P > 0 && max_blocks > 0, "attention: bad sizes");
    QE_REQUIRE(Hq % Hkv == 0, "attention: %d query heads are no multiple of %d key/value heads", Hq, Hkv);
    QE_REQUIRE(window >= 0, "attention: negative window");
    QE_REQUIRE(algo == 0 || algo == 1, "attention: unknown algo %d", algo);
    if (T == 0) return 0;
    return qe_attention_generic(q, out, cache, positions, tok_seq, block_table, max_blocks, T, Hq, Hkv,
                                D, P, scale, window, dt_a, stream);
}
