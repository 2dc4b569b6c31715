"""Pins the autotuner part of the oracle by hand-derived values: tile heuristic (constants and integer
arithmetic of the reference's Autotuner.cpp:571-655), link model, exec lookup, overlap models."""
import ctypes as C

import pytest

from oracle_binding import make_table, orc_link, orc_problem

TILE = 1024 * 1024 * 8  # bytes of a 1024^2 fp64 tile


def slowdowns(orc, D1, D2, D3, T, units=1):
    sl = (C.c_double * 6)()
    orc.orc_get_T_slowdowns(D1, D2, D3, units, T, sl)
    return list(sl)


def test_heuristic_known_answers(orc):
    """Worked by hand from the penalty terms (1 active unit): only the sub-kernel-count term 2/sk is non-zero for
    dividing tile sizes inside [2048, 4096]."""
    sl = (C.c_double * 6)()
    assert orc.orc_optimize_tile(16384, 16384, 16384, 1, sl) == 2048
    assert sl[0] == 0.00390625 and orc.orc_sk_num_blas3(16384, 16384, 16384, 2048) == 512
    assert orc.orc_optimize_tile(4096, 4096, 4096, 1, sl) == 2048
    assert sl[0] == 0.25 and orc.orc_sk_num_blas3(4096, 4096, 4096, 2048) == 8
    assert orc.orc_optimize_tile(32768, 32768, 32768, 1, sl) == 4096
    assert sl[0] == 0.00390625 and orc.orc_sk_num_blas3(32768, 32768, 32768, 4096) == 512
    assert orc.orc_optimize_tile(40000, 40000, 2048, 1, sl) == 2048
    # 40000 = 19*2048 + 1088: two non-dividing dims cost 1/19 each, 400 subkernels cost 2/400
    assert abs(sl[0] - (2.0 / 19 + 2.0 / 400)) < 1e-15 and abs(sl[2] - 2.0 / 19) < 1e-15 and sl[4] == 0.005
    assert orc.orc_sk_num_blas3(40000, 40000, 2048, 2048) == 400


def test_heuristic_terms(orc):
    # T below TILE_MIN: 2048/T * 0.2
    s = slowdowns(orc, 8192, 8192, 8192, 1024)
    assert s[3] == 0.4 and s[4] == 2.0 / 512 and s[5] == 0 and s[2] == 0
    # T above TILE_MAX: integer division T/4096 times 0.1
    s = slowdowns(orc, 16384, 16384, 16384, 8192)
    assert s[5] == 0.2 and s[4] == 2.0 / 8
    s = slowdowns(orc, 16384, 16384, 16384, 6000)
    assert s[5] == 0.1  # 6000/4096 -> 1
    # more than 512 subkernels: extra sk/512 * 0.1
    s = slowdowns(orc, 16384, 16384, 16384, 1024)
    assert abs(s[4] - (2.0 / 4096 + 4096 / 512 * 0.1)) < 1e-15
    # imbalance term with 3 units: bucket_num = Mg*Ng = 64, 64 % 3 = 1, 64 / 3 = 21 -> 1/21*3
    s = slowdowns(orc, 16384, 16384, 16384, 2048, units=3)
    assert abs(s[1] - 1.0 / 21 * 3) < 1e-15
    assert slowdowns(orc, 16384, 16384, 16384, 2048, units=1)[1] == 0.0
    assert abs(sum(s[1:]) - s[0]) < 1e-15


def test_block_num(orc):
    assert orc.orc_gemm_block_num(16384, 16384, 16384, 2048, 1) == 257  # 1 + 64 + 64 + 2*64
    assert orc.orc_gemm_block_num(16384, 16384, 16384, 2048, 0) == 193
    assert orc.orc_gemm_block_num(40000, 40000, 2048, 2048, 1) == 1 + 20 + 20 + 800


def test_link_model_closed_forms(orc):
    m1, m2 = orc_link(1e-5, 2e-11, 1.2), orc_link(2e-5, 2.5e-11, 1.5)
    assert abs(orc.orc_t_com_predict(m1, 1e6) - 3e-5) < 1e-18
    assert orc.orc_t_com_predict(m1, 0.0) == 0.0 and orc.orc_t_com_predict(m1, -1.0) == -1.0
    assert abs(orc.orc_t_com_sl(m1, 1e6) - 3.4e-5) < 1e-18
    # t_sl1 = 3.4e-5 < t_sl2 = 9.5e-5: t_sl1*(1 - 1/1.5) + 2e6*2.5e-11 + 2e-5/1.5
    assert abs(orc.orc_t_com_bid_predict(m1, m2, 1e6, 2e6) - (3.4e-5 / 3 + 5e-5 + 2e-5 / 1.5)) < 1e-18
    # swapped sizes take the other branch: t_sl1 = 1e-5 + 2e-11*4e6*1.2 = 1.06e-4 ; t_sl2 = 2e-5 + 2.5e-11*1e5*1.5 = 2.375e-5
    assert abs(orc.orc_t_com_bid_predict(m1, m2, 4e6, 1e5) - (2.375e-5 * (1 - 1 / 1.2) + 4e6 * 2e-11 + 1e-5 / 1.2)) < 1e-18
    assert orc.orc_t_com_bid_predict(m1, m2, 0.0, 2e6) == orc.orc_t_com_predict(m2, 2e6)
    assert orc.orc_t_com_bid_predict(m1, m2, 1e6, 0.0) == orc.orc_t_com_predict(m1, 1e6)
    # slowdown clamp when a Link-Stats file is read
    assert orc.orc_clamp_slowdown(0.5) == 1.0 and orc.orc_clamp_slowdown(3.0) == 2.0
    assert orc.orc_clamp_slowdown(1.03) == 1.0 and orc.orc_clamp_slowdown(1.4) == 1.4


def v100_table():
    # rows 8, 16, 24 of the reference's silver1 cublasDgemm_dev-0_TransA-N_TransB-N_1.1.log
    return make_table([2048, 4096, 8192], [2.556160e-03, 1.921535e-02, 1.578847e-01], "NNN", "NNN")


def test_exec_lookup(orc):
    tab, keep = v100_table()
    assert orc.orc_exec_predict(tab, 2048, b"N", b"N") == 2.556160e-03
    assert orc.orc_exec_predict(tab, 8192, b"N", b"N") == 1.578847e-01
    assert orc.orc_exec_nearest_T(tab, 100) == 2048      # below the table: the smallest entry
    assert orc.orc_exec_nearest_T(tab, 5000) == 4096     # otherwise the largest entry not above
    assert orc.orc_exec_nearest_T(tab, 8192) == 8192
    assert orc.orc_exec_nearest_T(tab, 20000) == 8192
    # a miss scales the nearest entry with the cube of the size ratio
    got = orc.orc_exec_predict(tab, 3000, b"N", b"N")
    assert abs(got - 2.556160e-03 * 27e9 / 2048 ** 3) < 1e-15
    assert orc.orc_exec_predict(tab, 2048, b"T", b"N") == -1.0  # no row with these flags


def synth_problem(remote=(1, 1, 1), t_recv=0.5e-3, t_send=0.25e-3, sl=(1.0, 1.0), D=(4096, 4096, 4096)):
    tab, keep = make_table([512, 1024, 2048, 4096], [1e-3 * (t / 1024.0) ** 3 for t in (512, 1024, 2048, 4096)], "NNNN", "NNNN")
    p = orc_problem()
    p.D1, p.D2, p.D3 = D
    p.dtype_sz = 8
    p.ta, p.tb = b"N", b"N"
    for i in range(3):
        p.remote[i] = remote[i]
        p.out_remote[i] = remote[i]
    p.h2d = orc_link(0.0, t_recv / TILE, sl[0])
    p.d2h = orc_link(0.0, t_send / TILE, sl[1])
    p.exec = C.pointer(tab)
    return p, (tab, keep)


def test_overlap_models_by_hand(orc):
    """4096^3, T = 1024 (64 subkernels), t_exec = 1 ms, tile H2D 0.5 ms, D2H 0.25 ms, all operands on the host."""
    p, keep = synth_problem()
    # baseline: max(1, max(3*0.5, 0.25)) ms * 63 + 1 + 1.5 + 0.25 ms
    assert abs(orc.orc_predict_blas3(3, p, 1024) - 0.09725) < 1e-12
    assert abs(orc.orc_predict_blas3(4, p, 1024) - 0.09725) < 1e-12   # data-location: everything remote, same
    assert abs(orc.orc_predict_blas3(5, p, 1024) - 0.09725) < 1e-12   # bidirectional with slowdown 1
    # reuse: one_over = 48 - 3 = 45, zero_over = 63 - 45 = 18, two_over = 0
    assert abs(orc.orc_predict_blas3(6, p, 1024) - 0.06575) < 1e-12
    # full / no overlap on the largest tile (4096): exec 64 ms, recv 3*16*0.5 ms, send priced like a receive 8 ms
    assert abs(orc.orc_predict_blas3(9, p, 1024) - 0.064) < 1e-12
    assert abs(orc.orc_predict_blas3(10, p, 1024) - 0.096) < 1e-12
    # C on the device: two inputs remote, no output to send
    q, keep2 = synth_problem(remote=(1, 1, 0))
    assert abs(orc.orc_predict_blas3(4, q, 1024) - 0.065) < 1e-12
    # device holds the majority: transfers are priced with the local (zero) link
    r, keep3 = synth_problem(remote=(1, 0, 0))
    assert abs(orc.orc_predict_blas3(4, r, 1024) - 0.064) < 1e-12


def test_reuse_model_branches(orc):
    # transfer slower than compute: pairs of remote inputs add two_over = 3 + 3 + 3
    p, keep = synth_problem(t_recv=2e-3, t_send=1e-3)
    assert abs(orc.orc_predict_blas3(6, p, 1024) - 0.125) < 1e-12
    # t_recv < t_exec < 2 t_recv: the extra D3/T = 4 two-transfer kernels
    q, keep2 = synth_problem(t_recv=0.6e-3, t_send=0.3e-3)
    assert abs(orc.orc_predict_blas3(6, q, 1024) - 0.0669) < 1e-12


def test_bidirectional_with_slowdowns(orc):
    p, keep = synth_problem(sl=(1.25, 1.5))
    # t_over = 0.375 ms * (1 - 0.8) + 1.5 ms = 1.575 ms
    assert abs(orc.orc_predict_blas3(5, p, 1024) - 0.101975) < 1e-12


def test_blas1_bidirectional_by_hand(orc):
    Ts = [1 << 16, 1 << 18, 1 << 20, 1 << 22]
    tab, keep = make_table(Ts, [1e-4 * t / float(1 << 18) for t in Ts])
    p = orc_problem()
    p.D1, p.D2, p.D3, p.dtype_sz = 1 << 20, 1, 1, 8
    p.remote[0] = p.remote[1] = 1
    p.h2d = orc_link(0.0, 0.5e-3 / TILE, 1.25)
    p.d2h = orc_link(0.0, 0.25e-3 / TILE, 1.5)
    p.exec = C.pointer(tab)
    ins, outs = (C.c_int * 2)(1, 1), (C.c_int * 2)(0, 1)
    assert abs(orc.orc_predict_blas1_bidirectional(p, 2, ins, outs, 1 << 18) - 1.21875e-3) < 1e-15


def test_model_driven_tile_search(orc):
    p, keep = synth_problem(D=(8192, 8192, 8192))
    pred = C.c_double()
    T = orc.orc_optimize_tile_model(6, p, C.byref(pred))
    cands = [t for t in (512, 1024, 2048, 4096)]
    times = {t: orc.orc_predict_blas3(6, p, t) for t in cands}
    best = min(times, key=times.get)
    # the scan starts from the first table entry but reports max(minT, 1024) unless a later entry is strictly better
    assert T == (best if best != 512 else 1024)
    assert pred.value == times[best]
    # a problem smaller than the smallest allowed tile: T = min dim, prediction 0
    q, keep2 = synth_problem(D=(600, 600, 600))
    assert orc.orc_optimize_tile_model(6, q, C.byref(pred)) == 600 and pred.value == 0.0
