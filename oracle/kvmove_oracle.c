/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the KV-block migration and swap path.
 *
 * Nothing shipped may link or call this file.  Only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg use it, and there only as the checker.
 *
 * The arithmetic of this path lives in SwiftTransformer (libst_pybinding.so), a
 * third-party library that DistServe clones at default-branch HEAD without pinning a
 * version (reference README.md:26-28, distserve/__init__.py:4-16) and that is not in
 * the reference tree.  The reference has no golden vector, known-answer test or fixture
 * for migration or swap.  Therefore the functions below restate the semantics that the
 * reference's own call sites and layout contract fix, and the tests pin them through
 * what the mathematics fixes (special cases that reduce to torch index_select /
 * index_copy_ / cat, an independently written brute-force loop nest on tiny shapes,
 * conservation and round-trip invariants).  With respect to the absent native op
 * itself: PARITY UNPINNED (no reference-held vector exists to compare against).
 *
 * Layout contract (distserve/worker.py:107-121): every pool is a contiguous 5-D array
 *     [num_blocks, layers_local, kv_heads_local, block_size, head_dim]
 * K and V are separate pools with identical shape.
 * Slice rule: pipeline rank p of P owns layers [p*L/P, (p+1)*L/P)
 * (distserve/config.py:279-286); tensor rank t of T owns KV heads [t*H/T, (t+1)*H/T)
 * (distserve/config.py:225-257, contiguous in-order split as in
 * distserve/downloader/converter.py:339-350).
 */
#include <stdint.h>
#include <string.h>

typedef struct kvo_geom {
    int64_t num_layers;   /* L, whole model */
    int64_t num_kv_heads; /* H, whole model (KV heads) */
    int64_t block_size;   /* B, tokens per block */
    int64_t head_dim;     /* D */
    int64_t dtype_bytes;  /* s */
    int64_t ctx_pp, ctx_tp;           /* context instance pipeline / tensor sizes */
    int64_t dec_pp, dec_tp;           /* decoding instance sizes */
    int64_t dec_pp_rank, dec_tp_rank; /* the decoding rank that pulls */
} kvo_geom;

/*
 * Migration of one pool kind (call once for K, once for V).
 * Follows the call at distserve/worker.py:250-267: for every pair
 * (ctx_idx[i], dec_idx[i]) and every (layer l, head h) of the decoding rank's
 * rectangle, copy the B*D*s-byte head slab from the context rank that owns (l, h).
 *
 * src_pools[p * ctx_tp + t] is the base of context rank (pp p, tp t)'s pool, each with
 * src_num_blocks blocks.  Returns 0, or a negative value for an argument error.
 */
int kvo_migrate(const kvo_geom *g, const void *const *src_pools, int64_t src_num_blocks,
                const int64_t *ctx_idx, const int64_t *dec_idx, int64_t n,
                void *dst_pool, int64_t dst_num_blocks)
{
    if (g->num_layers % g->ctx_pp || g->num_layers % g->dec_pp) return -1;
    if (g->num_kv_heads % g->ctx_tp || g->num_kv_heads % g->dec_tp) return -1;
    const int64_t Lc = g->num_layers / g->ctx_pp, Hc = g->num_kv_heads / g->ctx_tp;
    const int64_t Ld = g->num_layers / g->dec_pp, Hd = g->num_kv_heads / g->dec_tp;
    const int64_t slab = g->block_size * g->head_dim * g->dtype_bytes;
    const int64_t l_first = g->dec_pp_rank * Ld, h_first = g->dec_tp_rank * Hd;

    for (int64_t i = 0; i < n; ++i) {
        if (ctx_idx[i] < 0 || ctx_idx[i] >= src_num_blocks) return -2;
        if (dec_idx[i] < 0 || dec_idx[i] >= dst_num_blocks) return -3;
    }
    for (int64_t i = 0; i < n; ++i) {
        for (int64_t l = l_first; l < l_first + Ld; ++l) {
            for (int64_t h = h_first; h < h_first + Hd; ++h) {
                const int64_t p = l / Lc, t = h / Hc;
                const char *src = (const char *)src_pools[p * g->ctx_tp + t];
                const int64_t s_off = ((ctx_idx[i] * Lc + (l - p * Lc)) * Hc + (h - t * Hc)) * slab;
                const int64_t d_off = ((dec_idx[i] * Ld + (l - l_first)) * Hd + (h - h_first)) * slab;
                memcpy((char *)dst_pool + d_off, src + s_off, (size_t)slab);
            }
        }
    }
    return 0;
}

/*
 * Swap of one pool kind, following distserve/worker.py:269-311:
 * dst_pool[dst_ids[i]] = src_pool[src_ids[i]] for whole local block slabs of
 * slab_bytes each.  The direction (host->HBM or HBM->host) is the caller's choice of
 * which pool is which.
 */
int kvo_swap(const int64_t *src_ids, const int64_t *dst_ids, int64_t n,
             const void *src_pool, int64_t src_num_blocks,
             void *dst_pool, int64_t dst_num_blocks, int64_t slab_bytes)
{
    for (int64_t i = 0; i < n; ++i) {
        if (src_ids[i] < 0 || src_ids[i] >= src_num_blocks) return -2;
        if (dst_ids[i] < 0 || dst_ids[i] >= dst_num_blocks) return -3;
    }
    for (int64_t i = 0; i < n; ++i)
        memcpy((char *)dst_pool + dst_ids[i] * slab_bytes,
               (const char *)src_pool + src_ids[i] * slab_bytes, (size_t)slab_bytes);
    return 0;
}
