// hqmq_append_kv: the stages of an append for the K and the V tensor of a cache, stage by stage for both.
#include "common.h"

using namespace hqmq;

extern "C" int hqmq_append_kv(const hqmq_append_args *k, const hqmq_append_args *v, void *stream) {
    if (!k || !v) return HQMQ_ERR_NULL;
    hipStream_t st = (hipStream_t)stream;
    const hqmq_append_args *a[2] = {k, v};
    hqmq_quantize_args q[2] = {k->q, v->q};
    Med3xCall med[2];
    CompactCall cmp[2];
    const CompactCall *with_q[2] = {nullptr, nullptr};
    int n_med = 0;
    for (int i = 0; i < 2; i++) {
        if (!(a[i]->median_mult > 0.f)) continue;
        if (!q[i].flag_plane || !a[i]->thr) return HQMQ_ERR_NULL;
        if (q[i].T < 1) continue;                 // nothing to append: no statistics either
        q[i].thr = a[i]->thr;
        med[n_med] = Med3xCall{q[i].x, q[i].x_stride_b, q[i].x_stride_h, q[i].x_stride_t, q[i].dtype, q[i].B, q[i].H, q[i].T,
                               q[i].n_chunks, a[i]->median_mult, a[i]->med_workspace, a[i]->med_workspace_bytes,
                               a[i]->median, a[i]->thr, a[i]->n_out};
        cmp[n_med] = CompactCall{q[i].x, q[i].x_stride_b, q[i].x_stride_h, q[i].x_stride_t, q[i].dtype, q[i].B, q[i].H, q[i].T,
                                 q[i].n_chunks, q[i].flag_plane, q[i].t_cap, q[i].t_off, q[i].pos, a[i]->sideband,
                                 a[i]->sb_cap, a[i]->sb_tile_off, a[i]->sb_count, a[i]->overflow, a[i]->sb_coord,
                                 q[i].main_plane, q[i].aux_plane, q[i].scale_plane, 0, q[i].main_bits, q[i].aux_bits,
                                 (1 << q[i].radius_bits) - 1};
        if (layout_bits(q[i].secondary_size, q[i].radius_bits, &cmp[n_med].idx_bits, nullptr, nullptr)) return HQMQ_ERR_SHAPE;
        const int rc = check_compact(cmp[n_med]);
        if (rc) return rc;
        with_q[i] = &cmp[n_med];
        n_med++;
    }
    int rc = n_med ? med3x_calls(med, n_med, st) : HQMQ_OK;
    if (rc) return rc;
    // short appends: the quantize launch compacts as well; longer ones get the compaction kernels
    bool compacted[2];
    rc = quantize_two(&q[0], &q[1], with_q[0], with_q[1], compacted, st);
    if (rc) return rc;
    CompactCall rest[2];
    int n_rest = 0;
    for (int i = 0; i < 2; i++)
        if (with_q[i] && !compacted[i]) rest[n_rest++] = *with_q[i];
    return n_rest ? compact_calls(rest, n_rest, st) : HQMQ_OK;
}
