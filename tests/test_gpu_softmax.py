"""GPU parity: softmax, the categorical NLL gather and its backward, row and
n-d forms, through the C ABI against the oracle."""
import math

import numpy as np
import pytest

from gpu_util import F32, assert_bit_exact, assert_close, call, cfg, dev, empty, host

pytestmark = pytest.mark.gpu

ROW_ENTRY_POINTS = ["anode_gpu_softmax_packed_block_f32", "anode_gpu_softmax_packed_deterministic_f32"]


# ---- the reference's own known-answer tests (tests/test_gpu.rs:595-736) ----

@pytest.mark.parametrize("name", ROW_ENTRY_POINTS)
def test_ref_softmax_zeros_is_exactly_one_over_32(name):
    for rows in (1, 2):
        y = empty(32 * rows)
        call(name, 32, rows, dev(np.zeros(32 * rows, F32)), y)
        assert np.all(host(y) == F32(1.0) / F32(32.0))


def test_ref_softmax_cat_nll_known_answers(oracle):
    p = empty(64)
    call("anode_gpu_softmax_packed_block_f32", 32, 2, dev(np.zeros(64, F32)), p)
    nll = empty(2)
    call("anode_gpu_softmax_cat_nll_packed_f32", 32, 2, p, dev(np.array([12, 17], np.uint32)), nll)
    assert_close(host(nll), [math.log(32.0)] * 2, "nll", rel=1e-6)
    # out-of-range label: NaN, and a NaN batch sum (tests/test_gpu.rs:651-690)
    call("anode_gpu_softmax_cat_nll_packed_f32", 32, 2, p, dev(np.array([12, 42], np.uint32)), nll)
    h = host(nll)
    assert np.isfinite(h[0]) and np.isnan(h[1]) and np.isnan(h.sum())
    # adjoint of the batch sum (tests/test_gpu.rs:692-736): dx = 1/32 - [k == label], exactly
    dx = empty(64)
    call("anode_gpu_softmax_cat_nll_bwd_packed_f32", 32, 2, dev(np.ones(2, F32)), p,
         dev(np.array([12, 17], np.uint32)), dx)
    want = np.full((2, 32), F32(1.0) / F32(32.0), F32)
    want[0, 12] -= 1
    want[1, 17] -= 1
    assert_bit_exact(host(dx), want.ravel(), "softmax_cat_nll_bwd closed form")


# ---- row form ----

ROW_SHAPES = [(1, 5), (2, 7), (3, 1000), (10, 32), (19, 513), (32, 2), (33, 9), (64, 300), (65, 3), (100, 17),
              (128, 5), (129, 4), (1000, 256), (1024, 3), (1025, 2), (2048, 2), (2049, 3), (5000, 2), (40000, 1),
              # several 256-row tiles of the thread-per-row kernel, ragged last tile, even and odd K
              (10, 4000), (7, 777), (32, 600), (16, 257), (4, 1025), (5, 256), (31, 1023),
              # either side of the switch from lane groups over an LDS tile to one wave per row, 2 to 8 lanes per row
              (208, 70), (209, 70), (212, 33), (40, 1000), (96, 300), (130, 77), (200, 50),
              (224, 33), (225, 33), (232, 17), (239, 40), (240, 9), (241, 9), (250, 21), (255, 19), (256, 33), (257, 5),
              # every count of values per lane the tile kernel is built for, one to eight lanes per row
              (20, 300), (24, 100), (28, 70), (36, 300), (47, 70), (52, 90), (75, 50), (92, 64), (108, 40), (150, 33),
              (180, 41), (215, 37),
              # rows in registers that start at every distance from a 128-byte line (K = 4 * odd)
              (212, 40), (1012, 19), (2044, 9), (2052, 11), (4100, 9), (8196, 3),
              # few rows of 513 to 2048 classes: a workgroup per row (16-byte accesses), and its neighbours
              (516, 7), (1000, 256), (1024, 512), (1028, 512), (2048, 40), (1000, 513), (512, 7),
              # the limits of the workgroup-per-row register kernel
              (4096, 3), (4097, 2), (8192, 2), (8193, 1), (16384, 2), (16385, 1),
              # ... and of its 512-thread form (rows of 9217 to 16384 classes)
              (9216, 2), (9217, 2), (9220, 3), (12289, 3), (16380, 2),
              # workgroups of 1024 threads: rows in registers up to 32768 classes, streamed twice beyond
              (16388, 3), (20000, 3), (32764, 2), (32768, 2), (32769, 1), (32772, 3), (50257, 2), (65536, 2),
              (65540, 1), (100003, 1), (262148, 2),
              # more long rows than the streaming kernel has workgroups: each walks several rows, the next row's
              # first batch requested while the current row is written
              (32772, 1100), (33001, 1030)]


@pytest.mark.parametrize("K,R", ROW_SHAPES)
@pytest.mark.parametrize("name", ROW_ENTRY_POINTS)
def test_softmax_rows(oracle, name, K, R):
    print(f"case {name} K={K} R={R}", flush=True)
    g = np.random.default_rng(K * 7 + R)
    x = (2 * g.standard_normal(K * R)).astype(F32)
    for offset in (0, 3):
        y = empty(K * R, offset=offset)
        # both entry points must be right for any K, whatever cfg says (dispatch at src/ops_gpu.rs:6153)
        call(name, K, R, dev(x, offset), y, cfg=cfg(32, 16))
        p = host(y)
        assert_close(p, oracle.softmax(K, R, x, f64=True), f"softmax K={K}", abs_floor=1e-30)
        assert_close(p.reshape(R, K).astype(np.float64).sum(1), np.ones(R), "rows sum to one", rel=1e-5)


def test_softmax_rows_special_values(oracle):
    K, R = 8, 4
    x = np.zeros((R, K), F32)
    x[0, :] = -np.inf
    x[0, 3] = 1.0          # -inf entries get probability 0
    x[1, :] = [1e30, -1e30, 0, 5, 5, 5, 5, 5]
    x[2, 2] = np.nan       # a NaN poisons its row only (max ignores NaN, the sum does not)
    x[3, :] = 88.0         # no overflow: the max is subtracted first
    y = empty(K * R)
    call("anode_gpu_softmax_packed_block_f32", K, R, dev(x), y)
    p = host(y).reshape(R, K)
    want = oracle.softmax(K, R, x.ravel(), f64=True).reshape(R, K)
    assert_close(p, want, "special values", abs_floor=1e-30)
    assert p[0, 3] == 1.0 and np.all(p[0, [0, 1, 2, 4]] == 0)
    assert np.all(np.isnan(p[2])) and not np.any(np.isnan(p[[0, 1, 3]]))
    # the same rows through the one-workgroup-per-row kernel (K above the register limit)
    K2 = 3000
    x2 = np.full((3, K2), -np.inf, F32)
    x2[0, 7] = 2.0
    x2[1, :] = 0.5
    x2[1, 0] = -np.inf     # a leading -inf must not turn into NaN
    x2[2, :] = np.linspace(-50, 50, K2)
    y2 = empty(3 * K2)
    call("anode_gpu_softmax_packed_deterministic_f32", K2, 3, dev(x2), y2)
    assert_close(host(y2), oracle.softmax(K2, 3, x2.ravel(), f64=True), "block kernel special values", abs_floor=1e-30)


@pytest.mark.parametrize("K", [20000, 40004, 70001, 140000])
def test_softmax_long_rows_special_values(oracle, K):
    # rows of 1024-thread workgroups (in registers) and rows that are streamed in batches with a running maximum:
    # batches of nothing but -inf before, between and after the finite values, the maximum in the first or in the
    # last batch, a NaN in the part that is read twice, a row of nothing but -inf
    R = 9
    print(f"case long rows K={K}", flush=True)
    x = np.full((R, K), -np.inf, F32)
    x[0, K - 3] = 2.0
    x[1, :] = 0.5
    x[1, :K // 2] = -np.inf
    x[2, :] = np.linspace(-50, 50, K)
    x[3, :] = np.linspace(50, -50, K)
    x[4, :] = 1.0
    x[4, K - 1] = np.nan
    x[5, 5] = 3.0
    x[5, K // 2] = 3.0
    x[6, :] = 88.0
    x[7, :] = np.random.default_rng(K).standard_normal(K).astype(F32)
    x[7, K // 3] = 1e30
    # row 8 stays -inf throughout: NaN, as exp(-inf - -inf) is
    for offset in (0, 1):
        y = empty(K * R, offset=offset)
        call("anode_gpu_softmax_packed_deterministic_f32", K, R, dev(x, offset), y)
        p = host(y).reshape(R, K)
        want = oracle.softmax(K, R, x.ravel(), f64=True).reshape(R, K)
        assert_close(p, want, f"long rows K={K}", abs_floor=1e-30)
        assert p[0, K - 3] == 1.0 and np.count_nonzero(p[0]) == 1
        assert np.all(p[1, :K // 2] == 0)
        assert np.all(np.isnan(p[4])) and np.all(np.isnan(p[8]))
        assert p[5, 5] == 0.5 and p[5, K // 2] == 0.5
        assert p[7, K // 3] == 1.0
        assert not np.any(np.isnan(p[[0, 1, 2, 3, 5, 6, 7]]))


@pytest.mark.parametrize("K,R", [(32773, 5), (50257, 3), (40002, 4), (65536, 3),
                                 # shorter rows: every row kernel family with arrays that lie differently
                                 (10, 3000), (33, 700), (100, 300), (250, 100), (1000, 256), (1001, 30), (2048, 12),
                                 # rows in registers: every workgroup size, and the longest row that fits each
                                 (2050, 5), (4062, 3), (4063, 3), (8158, 2), (8159, 2), (12289, 3), (16350, 2), (16351, 2),
                                 (30522, 2), (32734, 2), (32735, 2)])
def test_softmax_rows_touch_nothing_but_their_rows(oracle, K, R):
    # Rows of more than 32768 classes that do not start on 16-byte boundaries are read and written in the array's
    # 16-byte groups where x and y start equally far from such a boundary: the groups at a row's ends are shared with
    # its neighbours, and with whatever lies before and after the array.  Guard bands around y (and dx) must come
    # back untouched, for every distance from a boundary, and also where x and y lie differently (4-byte accesses);
    # the same for the kernels of shorter rows, whose 16-byte forms need every array of the launch aligned.
    import torch
    g = np.random.default_rng(K + R)
    x = (2 * g.standard_normal(K * R)).astype(F32)
    want = oracle.softmax(K, R, x, f64=True)
    lab = g.integers(0, K, R).astype(np.uint32)
    dy = g.standard_normal(R).astype(F32)
    # (x and y alike within a 16-byte group but not within a 128-byte line: (1, 5), (3, 31))
    for off_x, off_y in [(0, 0), (1, 1), (2, 2), (3, 3), (1, 2), (0, 3), (1, 5), (3, 31)]:
        print(f"case long rows K={K} R={R} x+{off_x} y+{off_y}", flush=True)
        buf = torch.full((K * R + 64,), 12345.0, dtype=torch.float32, device="cuda")
        y = buf[16 + off_y:16 + off_y + K * R]
        # what lies before and after x must not count: NaN there would reach every probability of the row
        xbuf = torch.full((K * R + 64,), float("nan"), dtype=torch.float32, device="cuda")
        xd = xbuf[16 + off_x:16 + off_x + K * R]
        xd.copy_(torch.from_numpy(x))
        call("anode_gpu_softmax_packed_deterministic_f32", K, R, xd, y)
        whole = host(buf)
        assert np.all(whole[:16 + off_y] == 12345.0) and np.all(whole[16 + off_y + K * R:] == 12345.0)
        assert_close(whole[16 + off_y:16 + off_y + K * R], want, f"softmax K={K} x+{off_x} y+{off_y}", abs_floor=1e-30)
        # softmax + NLL + backward in one launch: dx lies like y
        buf2 = torch.full((K * R + 64,), 12345.0, dtype=torch.float32, device="cuda")
        dbuf = torch.full((K * R + 64,), 54321.0, dtype=torch.float32, device="cuda")
        y2, dx = buf2[16 + off_y:16 + off_y + K * R], dbuf[16 + off_y:16 + off_y + K * R]
        nll = empty(R)
        call("anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32", K, R, xd, dev(lab), dev(dy), y2, nll, dx)
        whole2, wholed = host(buf2), host(dbuf)
        assert np.all(whole2[:16 + off_y] == 12345.0) and np.all(whole2[16 + off_y + K * R:] == 12345.0)
        assert np.all(wholed[:16 + off_y] == 54321.0) and np.all(wholed[16 + off_y + K * R:] == 54321.0)
        assert_bit_exact(whole2[16 + off_y:16 + off_y + K * R], whole[16 + off_y:16 + off_y + K * R], "fused p")
        p = whole2[16 + off_y:16 + off_y + K * R]
        assert_bit_exact(wholed[16 + off_y:16 + off_y + K * R], oracle.softmax_cat_nll_bwd(K, R, dy, p, lab), "fused dx")
        assert_close(host(nll), oracle.softmax_cat_nll(K, R, p, lab, f64=True), "fused nll", abs_floor=1e-6)


@pytest.mark.parametrize("K,R", [(10, 32), (1000, 256), (7, 5), (1, 9), (300, 11)])
def test_softmax_cat_nll_and_bwd_rows(oracle, K, R):
    g = np.random.default_rng(K + R)
    x = (2 * g.standard_normal(K * R)).astype(F32)
    lab = g.integers(0, K, R).astype(np.uint32)
    if R > 4:
        lab[2] = K          # first out-of-range value
        lab[4] = 0xFFFFFFFF
    dy = g.standard_normal(R).astype(F32)
    old = g.standard_normal(K * R).astype(F32)
    for offset in (0, 1):
        p_d = empty(K * R, offset=offset)
        call("anode_gpu_softmax_packed_deterministic_f32", K, R, dev(x, offset), p_d)
        p = host(p_d)
        nll = empty(R, offset=offset)
        call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p_d, dev(lab, offset), nll)
        # label gather: the index is exact, so nll must equal -log of exactly that stored probability
        idx = oracle.softmax_cat_gather_index(K, R, lab)
        ok = idx != np.iinfo(np.uint64).max
        want = np.full(R, np.nan)
        want[ok] = -np.log(p.astype(np.float64)[idx[ok].astype(np.int64)])
        assert_close(host(nll), want, "nll gather", abs_floor=1e-6)
        assert_close(host(nll), oracle.softmax_cat_nll(K, R, p, lab, f64=True), "nll", abs_floor=1e-6)

        dx = empty(K * R, offset=offset)
        call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, dev(dy, offset), p_d, dev(lab, offset), dx)
        assert_bit_exact(host(dx), oracle.softmax_cat_nll_bwd(K, R, dy, p, lab), "nll bwd vs fp32")
        assert_close(host(dx), oracle.softmax_cat_nll_bwd(K, R, dy, p, lab, f64=True), "nll bwd", abs_floor=1e-7)
        dxa = dev(old, offset)
        call("anode_gpu_softmax_cat_nll_bwd_packed_accumulate_f32", K, R, dev(dy, offset), p_d, dev(lab, offset), dxa)
        assert_bit_exact(host(dxa), oracle.softmax_cat_nll_bwd(K, R, dy, p, lab, dx_in=old), "nll bwd acc vs fp32")


# ---- n-d form ----

ND_SHAPES = [(64, 19, 2), (4, 3, 5), (5, 3, 4), (1, 10, 6), (2048, 19, 2), (100, 1, 3), (36, 4, 2), (40, 8, 3),
             (28, 16, 2), (12, 24, 2), (16, 32, 2), (8, 33, 2), (8, 64, 3), (6, 100, 2), (4, 130, 2), (7, 40, 3),
             # several waves of pixel groups with a ragged last wave, few and many classes
             (1300, 19, 3), (516, 32, 5), (1028, 2, 3),
             # eight lanes per pixel group (33 to 256 classes with 16-byte accesses), and the streamed kernel beyond
             (20, 48, 3), (20, 64, 2), (24, 65, 2), (24, 128, 2), (24, 129, 2), (16, 200, 2), (8, 256, 3), (520, 40, 2),
             (8, 300, 2), (5, 257, 3), (64, 1000, 2), (7, 300, 2),
             # planes of 1024 pixels and more never go through the LDS tile: every register and streaming kernel,
             # 16-byte and 4-byte forms
             (1028, 8, 2), (1032, 24, 2), (1024, 32, 2), (1028, 33, 2), (1028, 48, 2), (1024, 64, 1), (1032, 65, 2),
             (1028, 100, 1), (1024, 128, 1), (1028, 129, 1), (1024, 192, 1), (1028, 200, 1), (1024, 256, 2),
             (1028, 300, 1), (1025, 19, 2), (1025, 40, 2), (1027, 100, 1), (1025, 130, 1), (1025, 257, 1),
             # the LDS tile (planes that are not whole 64-byte pieces, up to 64 classes, samples up to 32 KB) and
             # its neighbours: the largest sample and one class more, the longest plane, one sample per tile and
             # many, sample sizes that are and are not multiples of four floats or of the 32 banks
             (196, 32, 9), (196, 41, 5), (196, 42, 3), (1023, 8, 3), (1020, 8, 5), (1020, 9, 2), (127, 64, 3),
             (127, 65, 3), (49, 20, 70), (7, 9, 1000), (4, 8, 4100), (2, 16, 3000), (6, 6, 700), (3, 64, 50),
             (2, 2, 9000), (2, 1, 5000), (15, 7, 300),
             (512, 32, 3), (3, 5461, 2), (196, 64, 9), (196, 84, 3), (9, 455, 6), (2, 8192, 3),
             # tiles of all classes of a run of pixels in LDS (from 193 classes on, from 65 on planes under 1024 pixels):
             # ragged last tiles, one tile per plane, 16 to 256 pixels per tile, the largest class counts that fit
             # (472, 944) and one more
             (64, 300, 3), (16, 900, 2), (16, 944, 1), (16, 945, 1), (784, 100, 2), (196, 150, 2), (2048, 472, 1),
             (2048, 473, 1), (20, 70, 5), (256, 65, 2), (1024, 193, 1), (1056, 200, 2), (1000, 65, 2),
             # samples of up to 63 KB with a tile to themselves (more than 32 classes, planes that are not whole 64-byte
             # pieces), the largest that fits and one class more, and a short plane that the column tiles keep
             (196, 70, 3), (196, 82, 2), (196, 83, 2), (100, 100, 3), (36, 128, 3), (900, 17, 2), (252, 64, 2),
             # whole samples in registers (short planes of whole 16-byte groups, more than 32 classes): every form of
             # the kernel -- 256, 512 and 1024 threads with 8 and 16 slots each --, the most classes the largest
             # form holds at 49 pixel groups (320) and one more, which goes back to the other kernels
             (64, 33, 5), (100, 33, 3), (36, 256, 3), (400, 40, 2), (784, 40, 2), (196, 200, 2), (196, 300, 2),
             (196, 320, 1), (196, 321, 1),
             # column tiles over planes that are not whole 32-byte pieces (256 pixels and more, 65 to 128 classes,
             # too many pixel groups for a sample in registers), and one class more
             (676, 100, 1), (900, 65, 2), (1012, 128, 1), (900, 129, 1),
             # column tiles in registers (33 to 1024 classes, planes of 128 pixels and more):
             # the fewest and the most classes and one more, 32 slots per thread from 513 classes on, the shortest plane and the next shorter one, 8 and 16
             # slots per thread, ragged last tiles, planes that are and are not whole 128-byte lines
             (128, 33, 3), (124, 300, 2), (132, 512, 2), (1028, 513, 1), (900, 300, 1), (400, 200, 2), (4100, 40, 1),
             (196, 600, 2), (1024, 1024, 1), (1028, 1025, 1), (901, 700, 1), (16, 1024, 2), (64, 600, 2), (100, 513, 1),
             (2048, 257, 1), (1024, 512, 1), (324, 256, 2), (4096, 64, 1),
             # planes that are not whole 16-byte groups through the 16-byte kernels (the last group of a plane ends
             # with the plane): two lanes per group up to 32 classes where no LDS tile holds the sample, column tiles
             # in registers from 129 pixels on
             (1001, 19, 2), (1023, 9, 2), (2049, 2, 3), (4225, 21, 1), (1026, 32, 2), (129, 33, 3), (131, 512, 1),
             (4225, 64, 1), (1031, 300, 1), (49, 300, 3), (17, 129, 5), (121, 200, 2), (25, 512, 2), (15, 300, 2),
             # the backward pass walked flat over planes that are not whole 16-byte groups (from 64 pixels on, from 200
             # when accumulating): the shortest such planes and the next shorter ones, arrays whose last group is partial
             (513, 5, 3), (511, 5, 3), (515, 3, 1), (517, 1, 3), (65, 5, 7), (63, 5, 7), (201, 3, 5), (199, 3, 5),
             # planes of more than 131072 pixels: the backward pass gives a thread four pixels and walks their classes
             (131076, 5, 1), (131080, 19, 1), (131073, 3, 1)]


@pytest.mark.parametrize("P,C,N", ND_SHAPES)
def test_softmax_nd_all_symbols(oracle, P, C, N):
    print(f"case P={P} C={C} N={N}", flush=True)
    g = np.random.default_rng(P * 3 + C)
    n = P * C * N
    x = g.standard_normal(n).astype(F32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    lab[g.random(P * N) < 0.05] = 255 if C <= 255 else 0xFFFFFFFF  # ignore-index style labels
    dy = g.standard_normal(P * N).astype(F32)
    old = g.standard_normal(n).astype(F32)
    for offset in (0, 1):
        p_d = empty(n, offset=offset)
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, dev(x, offset), p_d)
        p = host(p_d)
        assert_close(p, oracle.softmax_nd(P, C, N, x, f64=True), "softmax_nd", abs_floor=1e-30)

        nll = empty(P * N, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, p_d, dev(lab, offset), nll)
        idx = oracle.softmax_nd_cat_gather_index(P, C, N, lab)
        ok = idx != np.iinfo(np.uint64).max
        want = np.full(P * N, np.nan)
        want[ok] = -np.log(p.astype(np.float64)[idx[ok].astype(np.int64)])
        assert_close(host(nll), want, "nd nll gather", abs_floor=1e-6)
        assert np.array_equal(np.isnan(host(nll)), lab >= C)

        dx = empty(n, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dev(dy, offset), p_d, dev(lab, offset), dx)
        assert_bit_exact(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab), "nd bwd vs fp32")
        assert_close(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab, f64=True), "nd bwd", abs_floor=1e-7)
        dxa = dev(old, offset)
        call("anode_gpu_softmax_nd_cat_nll_bwd_packed_accumulate_f32", P, C, N, dev(dy, offset), p_d,
             dev(lab, offset), dxa)
        assert_bit_exact(host(dxa), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab, dx_in=old), "nd bwd acc vs fp32")


@pytest.mark.parametrize("P,C,N", [(64, 19, 3), (196, 19, 5), (196, 70, 3), (64, 300, 2), (1056, 200, 1), (2048, 19, 2),
                                   (1028, 300, 1), (36, 128, 3), (196, 150, 2), (400, 40, 2), (784, 40, 1), (196, 200, 2), (900, 65, 1), (900, 300, 1),
                                   (2048, 257, 1), (1001, 19, 2), (1025, 100, 1)])
def test_softmax_nd_arrays_that_lie_differently(oracle, P, C, N):
    # every n-d kernel family with arrays at different element offsets from a 16-byte boundary: the 16-byte forms
    # need all of a launch's arrays aligned, and any mix must still give the 4-byte forms' (correct) results;
    # the plain and the fused entry points, and guard bands round the outputs
    import torch
    g = np.random.default_rng(P + 7 * C)
    n = P * C * N
    x = g.standard_normal(n).astype(F32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    dy = g.standard_normal(P * N).astype(F32)
    want = oracle.softmax_nd(P, C, N, x, f64=True)

    def guarded(count, off, fill):
        buf = torch.full((count + 40,), fill, dtype=torch.float32, device="cuda")
        return buf, buf[16 + off:16 + off + count]

    def intact(buf, count, off, fill):
        h = host(buf)
        return bool(np.all(h[:16 + off] == fill) and np.all(h[16 + off + count:] == fill))

    for off_x, off_y, off_dx, off_lab in [(0, 0, 0, 0), (0, 1, 0, 0), (1, 0, 0, 0), (0, 0, 2, 0), (0, 0, 0, 1), (3, 2, 1, 3)]:
        print(f"case P={P} C={C} N={N} offsets {off_x} {off_y} {off_dx} {off_lab}", flush=True)
        ybuf, y = guarded(n, off_y, 777.0)
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, dev(x, off_x), y)
        assert intact(ybuf, n, off_y, 777.0)
        assert_close(host(y), want, "softmax_nd", abs_floor=1e-30)
        y2buf, y2 = guarded(n, off_y, 777.0)
        dbuf, dx = guarded(n, off_dx, 555.0)
        nbuf, nll = guarded(P * N, off_lab, 333.0)
        call("anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32", P, C, N, dev(x, off_x), dev(lab, off_lab),
             dev(dy, off_lab), y2, nll, dx)
        assert intact(y2buf, n, off_y, 777.0) and intact(dbuf, n, off_dx, 555.0) and intact(nbuf, P * N, off_lab, 333.0)
        p = host(y2)
        assert_close(p, want, "fused softmax_nd", abs_floor=1e-30)
        assert_bit_exact(p, host(y), "fused p vs plain p, whatever the label / nll / dy / dx arrays' alignment")
        assert_close(host(nll), oracle.softmax_nd_cat_nll(P, C, N, p, lab, f64=True), "fused nll", abs_floor=1e-6)
        assert_bit_exact(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab), "fused dx vs fp32 of its own p")


@pytest.mark.parametrize("P,C,N,off", [(2, 1, 2053, 0), (3, 1, 1, 4), (2, 1, 1, 4), (3, 1, 2049, 0), (2, 1, 2053, 4),
                                       (1, 3, 1, 4), (1, 2, 4097, 0)])
def test_softmax_nd_tile_of_fewer_than_four_floats(oracle, P, C, N, off):
    # the LDS-tile kernel with a last tile (or an only tile) of fewer than four floats that does not start on a
    # 128-byte line: it has no 16-byte group of its own and must go through the element loop alone.  The arrays lie
    # `off` floats into their allocations (16-byte aligned either way), with guard bands; plain and fused entry points.
    import torch
    g = np.random.default_rng(P + 5 * N)
    n = P * C * N
    x = g.standard_normal(n).astype(F32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    dy = g.standard_normal(P * N).astype(F32)
    want = oracle.softmax_nd(P, C, N, x, f64=True)

    def guarded(count, fill):
        buf = torch.full((count + 64,), fill, dtype=torch.float32, device="cuda")
        return buf, buf[32 + off:32 + off + count]

    def intact(buf, count, fill):
        h = host(buf)
        return bool(np.all(h[:32 + off] == fill) and np.all(h[32 + off + count:] == fill))

    xbuf, xd = guarded(n, 0.0)
    xd.copy_(torch.from_numpy(x))
    ybuf, y = guarded(n, 777.0)
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, xd, y)
    assert intact(ybuf, n, 777.0)
    assert_close(host(y), want, "softmax_nd", abs_floor=1e-30)
    y2buf, y2 = guarded(n, 777.0)
    dbuf, dx = guarded(n, 555.0)
    nbuf, nll = guarded(P * N, 333.0)
    call("anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32", P, C, N, xd, dev(lab), dev(dy), y2, nll, dx)
    assert intact(y2buf, n, 777.0) and intact(dbuf, n, 555.0) and intact(nbuf, P * N, 333.0)
    p = host(y2)
    assert_bit_exact(p, host(y), "fused p vs plain p")
    assert_close(host(nll), oracle.softmax_nd_cat_nll(P, C, N, p, lab, f64=True), "fused nll", abs_floor=1e-6)
    assert_bit_exact(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab), "fused dx vs fp32 of its own p")


@pytest.mark.parametrize("P", [8, 36, 100, 1028, 2048])
@pytest.mark.parametrize("C", [3, 19, 40, 100, 200, 300])
def test_softmax_nd_special_values(oracle, C, P):
    # register-resident (2 or 8 lanes per pixel group up to 256 classes; one pixel per thread without 16-byte
    # accesses up to 128) and streaming kernels: -inf entries get probability 0, a NaN
    # poisons its pixel only, a pixel of +-1e30 and one of large equal values do not overflow, widely spread logits
    # keep their small probabilities to the relative bar.  P = 8 goes through the LDS tile up to 64 classes; P = 36
    # and 100 keep whole samples in registers from 100 and 40 classes on; P = 1028 and 2048 take column tiles in
    # registers from 40 classes on (planes that are not, and are, whole 128-byte lines).
    N = 2
    g = np.random.default_rng(C)
    x = g.standard_normal((N, C, P)).astype(F32)
    x[0, :, 0] = -np.inf
    x[0, 1, 0] = 1.0
    x[0, :, 1] = 5.0
    x[0, 0, 1], x[0, 1, 1] = 1e30, -1e30
    x[0, 2, 2] = np.nan
    x[0, :, 3] = 88.0
    x[0, :, 4] = np.linspace(-60, 8, C)
    x[1, :, 5] = np.linspace(-20, 20, C)
    x[1, :, 6] = -np.inf          # nothing but -inf: NaN, as exp(-inf - -inf) is
    x[1, :, 7] = -np.inf          # a NaN whose neighbours are all -inf still poisons its pixel
    x[1, C - 1, 7] = np.nan
    x[1, 0, 7] = 1.0
    for offset in (0, 1):
        y = empty(x.size, offset=offset)
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, dev(x, offset), y)
        p = host(y).reshape(N, C, P)
        want = oracle.softmax_nd(P, C, N, x.ravel(), f64=True).reshape(N, C, P)
        assert_close(p, want, f"n-d special values C={C}", abs_floor=1e-30)
        assert p[0, 1, 0] == 1.0 and np.all(np.delete(p[0, :, 0], 1) == 0)
        assert np.all(np.isnan(p[0, :, 2])) and np.all(np.isnan(p[1, :, 6]))
        assert not np.any(np.isnan(np.delete(p.reshape(N * C, P), [2], axis=1)[:C]))
        assert np.all(p[0, :, 3] == p[0, 0, 3]) and abs(float(p[0, 0, 3]) * C - 1) < 1e-6


@pytest.mark.parametrize("P,C,N", [(64, 19, 3), (1025, 19, 2), (1025, 100, 1), (1028, 100, 1), (196, 100, 2), (7, 9, 50),
                                   (2049, 2, 2), (400, 300, 1)])
def test_softmax_nd_in_place(oracle, P, C, N):
    # y == x, as the reference's kernels allow (a thread reads nothing but the pixels it writes).  Planes that are
    # not whole 16-byte groups then keep their kernels with one pixel per thread: the 16-byte kernels let the last
    # two groups of such a plane overlap, which needs separate arrays.
    g = np.random.default_rng(P + C)
    n = P * C * N
    x = g.standard_normal(n).astype(F32)
    want = oracle.softmax_nd(P, C, N, x, f64=True)
    for offset in (0, 1):
        xd = dev(x, offset)
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, xd, xd)
        assert_close(host(xd), want, "softmax_nd in place", abs_floor=1e-30)

