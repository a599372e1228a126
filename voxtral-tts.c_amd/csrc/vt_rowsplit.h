/*
 * vt_rowsplit.h - how the rows of a decode phase are dealt to the workgroups of a grid, and which
 * workgroups an attention workgroup depends on.  Pure integer functions, compiled for the device by
 * hipcc and for the host by any C++ compiler: the narrow hand-overs around the decode attention
 * (vt_decode.hip) are only safe while the producer list below and the row split of the q|k|v phase
 * are the same function of the grid, so both are derived from vt_rows_per_wg() here, and a host
 * test walks every legal grid.
 */
#ifndef VT_ROWSPLIT_H
#define VT_ROWSPLIT_H

#ifdef __HIPCC__
#define VT_HD __host__ __device__ __forceinline__
#else
#define VT_HD static inline
#endif

/* Model dimensions of the backbone / acoustic transformer layer (voxtral_tts.h:19-27). */
#define VT_DIM      3072
#define VT_HEADS    32
#define VT_KV_HEADS 8
#define VT_HEAD_DIM 128
#define VT_Q_DIM    4096
#define VT_KV_DIM   1024
#define VT_QKV_DIM  6144
#define VT_FFN      9216

/* Rows per workgroup when n_rows rows go to G workgroups as contiguous blocks of a multiple of `align`
 * rows (the last workgroups may own fewer rows, or none). */
VT_HD int vt_rows_per_wg(int n_rows, int align, int G) {
    const int per = (n_rows + G - 1) / G;
    return (per + align - 1) / align * align;
}

/* q|k|v phase: rows in pairs (RoPE rotates adjacent rows) */
#define VT_QKV_ALIGN 2
VT_HD int vt_qkv_rows_per_wg(int G) { return vt_rows_per_wg(VT_QKV_DIM, VT_QKV_ALIGN, G); }

/* Direct attention schedule: workgroup wg serves query head `head` of kv head `kvh` and takes share
 * `part` of the positions.  The four workgroups of a kv head have the same wg % 8, i.e. one XCD. */
VT_HD void vt_attn_direct_map(int wg, int *kvh, int *head, int *part) {
    const int idx = wg / VT_KV_HEADS;
    *kvh = wg % VT_KV_HEADS;
    *head = *kvh * 4 + (idx & 3);
    *part = idx >> 2;
}

/* First q|k|v row of the three row ranges attention workgroup wg reads: the 128 q rows of its head, the
 * new K row and the new V row of its kv head. */
VT_HD int vt_attn_range_first(int wg, int k) {
    int kvh, head, part;
    vt_attn_direct_map(wg, &kvh, &head, &part);
    return k == 0 ? head * VT_HEAD_DIM : k == 1 ? VT_Q_DIM + kvh * VT_HEAD_DIM : VT_Q_DIM + VT_KV_DIM + kvh * VT_HEAD_DIM;
}

/* Number of workgroups that own q|k|v rows which attention workgroup wg of a G-workgroup grid reads
 * (a workgroup that owns rows of two ranges is counted twice). */
VT_HD int vt_attn_producer_count(int G, int wg) {
    const int per = vt_qkv_rows_per_wg(G);
    int n = 0;
    for (int k = 0; k < 3; k++) {
        const int f = vt_attn_range_first(wg, k);
        n += (f + VT_HEAD_DIM - 1) / per - f / per + 1;
    }
    return n;
}

/* The i-th of them (past the last one: the first again). */
VT_HD int vt_attn_producer_of(int G, int wg, int i) {
    const int per = vt_qkv_rows_per_wg(G);
    int j = i;
    for (int k = 0; k < 3; k++) {
        const int f = vt_attn_range_first(wg, k);
        const int w0 = f / per, n = (f + VT_HEAD_DIM - 1) / per - w0 + 1;
        if (j < n) return w0 + j;
        j -= n;
    }
    return vt_attn_range_first(wg, 0) / per;
}

#endif /* VT_ROWSPLIT_H */
