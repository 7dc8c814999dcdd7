/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 * Plain-C restatement of the integer-exact steps of the reference's MoE path
 * (router selection, expert sort).  It is a second, independent implementation
 * next to oracle/moe_oracle.py: tests cross-check the two and use this one where
 * numpy would be slow.  Only tests/, __graft_entry__ and bench.py's cpu_baseline
 * leg may load it.  Citations are relative to the reference tree.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* Router: softmax + top-k on raw logits, strict '>' scan in ascending expert
 * order, so ties go to the lowest index (src/topk_softmax_kernels.hip:23-64);
 * weights exp(x-max)/sum, divided by the sum of the selected ones when
 * renormalize (layers/moe/fused_moe.py:161-162).  The scan is run k times with
 * already selected experts excluded, which for k = 2 selects what the
 * reference's single pass selects. */
int oracle_topk_softmax(const float* logits, int64_t T, int E, int k, int renormalize,
                        float* weights, int32_t* ids) {
    if (E < 1 || k < 1 || k > E || E > 1024) return -1;
    unsigned char* used = (unsigned char*)malloc((size_t)E);
    if (!used) return -2;
    for (int64_t t = 0; t < T; ++t) {
        const float* row = logits + t * E;
        float mx = -INFINITY;
        for (int e = 0; e < E; ++e) mx = row[e] > mx ? row[e] : mx;
        float sum = 0.0f;
        for (int e = 0; e < E; ++e) sum += expf(row[e] - mx);
        memset(used, 0, (size_t)E);
        float sel = 0.0f;
        for (int j = 0; j < k; ++j) {
            int best = -1;
            for (int e = 0; e < E; ++e) {
                if (used[e]) continue;
                if (best < 0 || row[e] > row[best]) best = e;
            }
            used[best] = 1;
            ids[t * k + j] = best;
            weights[t * k + j] = expf(row[best] - mx) / sum;
            sel += weights[t * k + j];
        }
        if (renormalize)
            for (int j = 0; j < k; ++j) weights[t * k + j] /= sel;
    }
    free(used);
    return 0;
}

/* Expert sort: count, pad every expert to a multiple of block, exclusive
 * cumsum, stable scatter, block->expert table
 * (src/moe_align_block_size.hip:78-135); sorted ids start as -1 and expert_ids
 * as 0 (layers/moe/moe_align_block_size.py:32-48). */
int oracle_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int E, int block,
                                int32_t* sorted_ids, int64_t sorted_len, int32_t* expert_ids,
                                int64_t expert_ids_len, int32_t* post_pad) {
    if (E < 1 || block < 1) return -1;
    int64_t* cnt = (int64_t*)calloc((size_t)E, sizeof(int64_t));
    int64_t* off = (int64_t*)calloc((size_t)E + 1, sizeof(int64_t));
    if (!cnt || !off) { free(cnt); free(off); return -2; }
    for (int64_t i = 0; i < sorted_len; ++i) sorted_ids[i] = -1;
    for (int64_t i = 0; i < expert_ids_len; ++i) expert_ids[i] = 0;
    for (int64_t i = 0; i < numel; ++i)
        if (topk_ids[i] >= 0 && topk_ids[i] < E) ++cnt[topk_ids[i]];
    for (int e = 0; e < E; ++e) off[e + 1] = off[e] + (cnt[e] + block - 1) / block * block;
    post_pad[0] = (int32_t)off[E];
    for (int e = 0; e < E; ++e)
        for (int64_t p = off[e]; p < off[e + 1]; p += block)
            if (p / block < expert_ids_len) expert_ids[p / block] = e;
    memset(cnt, 0, (size_t)E * sizeof(int64_t));
    for (int64_t i = 0; i < numel; ++i) {
        const int32_t e = topk_ids[i];
        if (e < 0 || e >= E) continue;
        const int64_t pos = off[e] + cnt[e]++;
        if (pos < sorted_len) sorted_ids[pos] = (int32_t)i;
    }
    free(cnt);
    free(off);
    return 0;
}
