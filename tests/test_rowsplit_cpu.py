"""The narrow hand-overs around the decode attention (vt_decode.hip) wait only for the workgroups
that vt_attn_producer_of() names.  That is safe only while those lists, taken over all attention
workgroups, cover every workgroup that owns q|k|v rows in the row split of the q|k|v phase, for
every grid the kernel accepts.  The two are the same integer functions on the host and on the
device (vt_rowsplit.h); this test compiles the header with g++ and walks every legal grid."""
import os
import subprocess

import numpy as np

import vtsupport as S

CSRC = os.path.join(S.ROOT, "voxtral-tts.c_amd", "csrc")

PROG = r"""
#include <stdio.h>
#include "vt_rowsplit.h"
int main(void) {
    for (int G = 72; G <= 256; G += 8) {
        const int per = vt_qkv_rows_per_wg(G);
        printf("G %d per %d\n", G, per);
        for (int wg = 0; wg < G; wg++) {
            int kvh, head, part;
            vt_attn_direct_map(wg, &kvh, &head, &part);
            const int n = vt_attn_producer_count(G, wg);
            printf("wg %d %d %d %d n %d :", wg, kvh, head, part, n);
            for (int i = 0; i < 64; i++) printf(" %d", vt_attn_producer_of(G, wg, i));
            printf("\n");
        }
    }
    return 0;
}
"""


def run_prog(tmp_path):
    src = tmp_path / "rowsplit.cc"
    src.write_text(PROG)
    exe = tmp_path / "rowsplit"
    subprocess.check_call(["g++", "-O1", "-I", CSRC, "-o", str(exe), str(src)])
    return subprocess.check_output([str(exe)], text=True).splitlines()


def test_attention_producers_cover_every_row_owner(tmp_path):
    lines = run_prog(tmp_path)
    G = per = None
    grids = {}
    for ln in lines:
        f = ln.split()
        if f[0] == "G":
            G, per = int(f[1]), int(f[3])
            grids[G] = {"per": per, "wgs": {}}
        else:
            wg, kvh, head, part, n = int(f[1]), int(f[2]), int(f[3]), int(f[4]), int(f[6])
            grids[G]["wgs"][wg] = (kvh, head, part, n, [int(v) for v in f[8:]])
    assert sorted(grids) == list(range(72, 257, 8))
    for G, g in grids.items():
        per = g["per"]
        # the row split itself: contiguous blocks of `per` rows, per even, all 6144 rows covered
        assert per % 2 == 0 and per * G >= 6144 and (per - 2) * G < 6144 + 2 * G
        owners = {wg for wg in range(G) if wg * per < 6144}
        owner_of = lambda row: row // per
        for wg, (kvh, head, part, n, lst) in g["wgs"].items():
            assert kvh == wg % 8 and head == kvh * 4 + (wg // 8) % 4 and part == wg // 32
            assert 3 <= n <= 64, (G, wg, n)                       # one poll lane per producer
            # exactly the owners of the rows this workgroup reads: q rows of its head, new K and V rows of its kv head
            want = set()
            for first in (head * 128, 4096 + kvh * 128, 5120 + kvh * 128):
                want |= {owner_of(r) for r in range(first, first + 128)}
            assert set(lst[:n]) == want, (G, wg)
            assert all(v == lst[0] for v in lst[n:])              # lanes past the end watch the first one again
            assert want <= owners
        # every schedule's attention workgroups (32 x 1, 2 or 8 parts) wait, between them, for every owner
        for busy in (32, 64, 256):
            if busy > G:
                continue
            seen = set()
            for wg in range(busy):
                n, lst = g["wgs"][wg][3], g["wgs"][wg][4]
                seen |= set(lst[:n])
            assert seen == owners, (G, busy, sorted(owners - seen))


def test_rows_per_workgroup_matches_the_phases(tmp_path):
    # the split the kernels use for their four phases on the full grid: 24 / 12 / 72 / 12 rows
    src = tmp_path / "per.cc"
    src.write_text('#include <stdio.h>\n#include "vt_rowsplit.h"\nint main(){printf("%d %d %d %d\\n",'
                   'vt_rows_per_wg(VT_QKV_DIM,2,256),vt_rows_per_wg(VT_DIM,1,256),vt_rows_per_wg(2*VT_FFN,2,256),'
                   'vt_rows_per_wg(VT_DIM,1,200));return 0;}')
    exe = tmp_path / "per"
    subprocess.check_call(["g++", "-I", CSRC, "-o", str(exe), str(src)])
    assert subprocess.check_output([str(exe)], text=True).split() == ["24", "12", "72", "16"]
