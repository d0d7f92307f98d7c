"""CPU checks of the launch planners: they size rounds of workgroups by the number of compute units
the machine reports (a full MI355X has 256 in 8 dies; its partitions and other parts of the family
have 64, 128, 304, ...), not by a constant.  The planners run on the host, so no device is needed:
`t2sp_set_machine` states the machine and the `*_plan` calls of include/t2sp_hip.h return what would
be launched."""
import ctypes

import pytest

import t2sp_amd

CUS = [64, 128, 256, 304]


@pytest.fixture
def lib():
    L = t2sp_amd.lib()
    i32p = ctypes.POINTER(ctypes.c_int)
    L.t2sp_set_machine.argtypes = [ctypes.c_int, ctypes.c_int]
    L.t2sp_set_machine.restype = None
    L.t2sp_sgemm_plan.argtypes = [ctypes.c_int] * 3 + [i32p, i32p]
    L.t2sp_conv2d_plan.argtypes = [ctypes.c_int] * 3 + [i32p]
    L.t2sp_ssyrk_plan.argtypes = [ctypes.c_int] * 3 + [i32p]
    L.t2sp_capsule_direct16_plan.argtypes = [ctypes.c_int] * 2 + [i32p]
    yield L
    L.t2sp_set_machine(0, 0)          # back to asking the device


@pytest.mark.parametrize("cus,xcds", [(64, 2), (128, 4), (256, 8), (304, 8), (32, 1), (38, 1), (152, 4), (76, 2)])
def test_dies_follow_from_the_compute_units(lib, cus, xcds):
    lib.t2sp_set_machine(cus, 0)
    assert (lib.t2sp_machine_cus(), lib.t2sp_machine_xcds()) == (cus, xcds)
    lib.t2sp_set_machine(cus, 3)
    assert lib.t2sp_machine_xcds() == 3


@pytest.mark.parametrize("cus", CUS)
@pytest.mark.parametrize("shape", [(8192, 8192, 8192), (6144, 6144, 6144), (5120, 5120, 2048), (4096, 16384, 2048),
                                   (10240, 10240, 1024), (7168, 7168, 7168), (114688, 128, 288), (5120, 5120, 256)])
def test_sgemm_launches_whole_rounds_then_a_split_rest(lib, cus, shape):
    lib.t2sp_set_machine(cus, 0)
    M, N, K = shape
    edge, ph = ctypes.c_int(0), (ctypes.c_int * 12)()
    n = lib.t2sp_sgemm_plan(M, N, K, ctypes.byref(edge), ph)
    assert n >= 1 and edge.value in (128, 256)
    tiles = -(-M // edge.value) * -(-N // edge.value)
    phases = [(ph[3 * i], ph[3 * i + 1], ph[3 * i + 2]) for i in range(n)]
    covered = 0
    for i, (first, count, splits) in enumerate(phases):
        assert first == covered and count > 0 and splits >= 1
        covered += count
        if splits > 1:
            assert count * splits <= cus            # a split rest is at most one round of workgroups
        elif i == 0 and tiles >= cus and n > 1:
            assert count % cus == 0                 # the unsplit part is whole rounds
    assert covered == tiles
    # (a rest of more than half a round saves too little to repay its planes and second launch, and so does
    # any rest under a short reduction: then everything goes as one launch)
    if tiles % cus and tiles > cus and K >= 2048 and tiles % cus <= cus // 2:
        assert any(s > 1 for _, _, s in phases), (cus, phases)
    if tiles > cus and K <= 384:
        assert phases == [(0, tiles, 1)], (cus, phases)


@pytest.mark.parametrize("cus", CUS)
def test_conv_stages_are_whole_rounds_until_the_rest(lib, cus):
    """The benchmark convolution: CO = 256, 64 x 56 x 56 output pixels, reduction 2304."""
    lib.t2sp_set_machine(cus, 0)
    CO, P, KRED = 256, 64 * 56 * 56, 2304
    st = (ctypes.c_int * 16)()
    n = lib.t2sp_conv2d_plan(CO, P, KRED, st)
    assert n >= 1
    edge = {1: (256, 256), 2: (128, 128), 3: (64, 128)}
    p = 0
    for i in range(n):
        cfg, p0, p1, splits = st[4 * i], st[4 * i + 1], st[4 * i + 2], st[4 * i + 3]
        bm, bn = edge[cfg]
        assert p0 == p and p1 > p0
        tiles = -(-CO // bm) * -(-(p1 - p0) // bn)
        if i < n - 1:
            assert splits == 1 and tiles % cus == 0, (cus, i, tiles)
        p = p1
    assert p == P


@pytest.mark.parametrize("cus", CUS)
def test_conv_rest_never_puts_two_or_three_two_wave_workgroups_on_a_cu(lib, cus):
    """Convolutions too small for whole rounds.  A CU hands out its SIMDs in a cycle that moves on by one per
    workgroup, so two or three workgroups of two waves (64 x 128 tiles) load one SIMD twice and take as long as
    four; one alone runs at half the CU's rate.  A plan with two or three of them per CU is therefore never
    the cheapest unless a split reduction makes them that many: unsplit, one per CU or at least four cost less."""
    lib.t2sp_set_machine(cus, 0)
    st = (ctypes.c_int * 16)()
    edge = {1: (256, 256), 2: (128, 128), 3: (64, 128)}
    for CO, P, KRED in ((256, 32 * 14 * 16, 2304), (250, 8 * 28 * 28, 2304), (144, 16 * 28 * 28, 1296), (512, 16 * 7 * 8, 4608),
                        (64, 32 * 30 * 32, 576), (64, 8 * 30 * 32, 1152), (48, 40 * 30 * 32, 576), (64, 50 * 30 * 32, 2304)):
        n = lib.t2sp_conv2d_plan(CO, P, KRED, st)
        cfg, p0, p1, splits = st[4 * (n - 1)], st[4 * (n - 1) + 1], st[4 * (n - 1) + 2], st[4 * (n - 1) + 3]
        bm, bn = edge[cfg]
        groups = -(-CO // bm) * -(-(p1 - p0) // bn) * splits
        per_cu = -(-groups // cus)
        if cfg == 3:
            # (two or three per CU only as the deepest split a short reduction allows)
            assert per_cu == 1 or per_cu >= 4 or splits > 1, (cus, CO, P, KRED, cfg, splits, per_cu)


def test_conv_takes_the_one_launch_form_for_small_convolutions_only(lib):
    """On the full machine: the benchmark convolution and other many-round shapes keep the staged LDS-tile
    plan, small and middle-sized ones with a reduction of more than 288 rows take the 16 x 16 form, shorter
    reductions only with up to 64 output channels (where the LDS tiles are the two-wave ones, which a CU
    runs one workgroup after the other) and up to two or three tiles per CU; its tiles cover CO with at
    most 6 row blocks."""
    lib.t2sp_set_machine(256, 8)
    lib.t2sp_conv2d_direct16_plan.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_void_p]
    out, times = (ctypes.c_int * 4)(), (ctypes.c_double * 2)()

    def takes(N, CI, CO, OH, OW, KH=3):
        P, K = N * OH * ((OW + 3) // 4 * 4), CI * KH * KH
        r = lib.t2sp_conv2d_direct16_plan(CO, P, K, out, times)
        mb, rpt, tm, tn = out
        assert 1 <= mb <= 6 and rpt <= 16 * mb and tm * rpt >= CO and tn * 64 >= P
        assert times[0] > 0 and times[1] > 0
        return r

    assert not takes(64, 256, 256, 56, 56)
    assert not takes(64, 512, 512, 28, 28)
    assert not takes(64, 64, 256, 56, 56, 1)
    for shape in ((32, 64, 64, 30, 30), (8, 256, 256, 14, 14), (16, 144, 144, 28, 28), (4, 128, 128, 28, 28), (1, 256, 256, 56, 56)):
        assert takes(*shape), shape
    # up to 64 output channels: measured against the 64 x 128 LDS tiles at 64..1536 tiles and four reductions
    for shape in ((1, 64, 64, 224, 224), (16, 32, 64, 64, 64), (4, 64, 64, 56, 56, 1), (2, 16, 32, 128, 128), (24, 32, 64, 64, 64)):
        assert takes(*shape), shape
    for shape in ((128, 32, 64, 64, 64), (24, 64, 64, 64, 64, 1), (64, 32, 64, 64, 64)):
        assert not takes(*shape), shape
    lib.t2sp_set_machine(0, 0)


@pytest.mark.parametrize("cus", CUS)
def test_syrk_splits_only_a_small_last_round(lib, cus):
    lib.t2sp_set_machine(cus, 0)
    out = (ctypes.c_int * 3)()
    for N in (4096, 8192, 12288):
        assert lib.t2sp_ssyrk_plan(N, 8192, 256, out) == 1
        total, tail, splits = out[0], out[1], out[2]
        side = N // 256
        assert total == side * (side + 1) // 2
        if splits > 1:
            assert tail == total % cus and 0 < tail <= cus // 2 and tail * splits <= cus
        else:
            assert tail == 0


@pytest.mark.parametrize("cus", CUS)
def test_capsule_direct_tiles_fill_rounds_of_the_machine(lib, cus):
    """The benchmark capsule layer: 32 x 49 pixels x 4 rows = 6272 vote rows by 128 columns."""
    lib.t2sp_set_machine(cus, 0)
    out = (ctypes.c_int * 6)()
    assert lib.t2sp_capsule_direct16_plan(6272, 128, out) == 1
    rpt, mb, nb, tiles_m, tiles_n, rounds = list(out)
    assert rpt % 4 == 0 and mb == -(-rpt // 16) and tiles_m == -(-6272 // rpt) and tiles_n == -(-128 // (16 * nb))
    groups = tiles_m * tiles_n
    assert (rounds - 1) * cus < groups <= rounds * cus
    assert groups > rounds * cus * 0.9              # the last round is nearly full


def test_unguarded_loop_bodies_only_fetch_whole_k_tiles():
    """The body of k-tile t fetches tile t + 2 (16 deep) without a guard when t is below
    t2sp_sgemm_tail_from(k_len): every such fetch must end inside the reduction, for any length;
    and from 64 on all but the last two pairs of tiles are unguarded."""
    L = t2sp_amd.lib()
    L.t2sp_sgemm_tail_from.argtypes = [ctypes.c_int]
    for k_len in list(range(0, 600)) + [8192, 8196, 8200, 8220, 8223, 100000, 100001]:
        t = L.t2sp_sgemm_tail_from(k_len)
        assert t >= 0 and t % 2 == 0
        if t > 0:
            # the last unguarded pair of bodies is (t - 2, t - 1): it fetches tiles t and t + 1
            assert (t + 2) * 16 <= k_len
        tiles = -(-k_len // 16)
        if k_len >= 64:
            assert t >= tiles - 5


def test_planners_take_extreme_extents(lib):
    """Every planner and workspace query with extents from 1 up to 2^31 - 1, in random combinations: each must
    return (0 / no plan beyond T2SP_MAX_EXTENT = 2^30 per dimension) without overflowing its 32-bit tile arithmetic
    or looping for long.  `make -C t2sp_amd/csrc asan-check` runs this under UndefinedBehaviorSanitizer, which is
    what turns an overflow into a failure; it found four, all fixed."""
    import random
    import time
    L = lib
    L.t2sp_set_machine(256, 8)
    i32, sz = ctypes.c_int, ctypes.c_size_t
    for f in (L.t2sp_sgemm_workspace_bytes, L.t2sp_sgemm_ex_workspace_bytes, L.t2sp_conv2d_workspace_bytes,
              L.t2sp_ssyrk_workspace_bytes, L.t2sp_mttkrp_workspace_bytes, L.t2sp_capsule_workspace_bytes):
        f.restype = sz
    L.t2sp_sgemm_workspace_bytes.argtypes = [i32] * 3
    L.t2sp_sgemm_ex_workspace_bytes.argtypes = [i32] * 4
    L.t2sp_conv2d_workspace_bytes.argtypes = [i32] * 7
    L.t2sp_ssyrk_workspace_bytes.argtypes = [i32] * 3
    L.t2sp_mttkrp_workspace_bytes.argtypes = [i32] * 6
    L.t2sp_conv2d_direct16_plan.argtypes = [i32] * 3 + [ctypes.POINTER(i32), ctypes.POINTER(ctypes.c_double)]
    rng = random.Random(1)
    edge = [1, 2, 3, 4, 15, 16, 17, 63, 64, 65, 127, 128, 255, 256, 257, 1023, 4096, 65535, 65536, 1 << 20,
            (1 << 22) - 1, 1 << 22, 1 << 30, (1 << 30) + 1, (1 << 31) - 1]

    def pick():
        return rng.choice(edge) if rng.random() < 0.7 else rng.randint(1, 1 << 20)

    t0 = time.time()
    for _ in range(3000):
        M, N, K = pick(), pick(), pick()
        te, ph = i32(), (i32 * 12)()
        n = L.t2sp_sgemm_plan(M, N, K, ctypes.byref(te), ph)
        assert 0 <= n <= 4 and (max(M, N, K) <= 1 << 30 or n == 0)
        if max(M, N, K) > 1 << 30:
            assert L.t2sp_sgemm_workspace_bytes(M, N, K) == 0
        else:
            L.t2sp_sgemm_workspace_bytes(M, N, K)
        L.t2sp_sgemm_ex_workspace_bytes(rng.randint(0, 1), M, N, K)
        assert 0 <= L.t2sp_conv2d_plan(pick(), pick(), pick(), (i32 * 16)()) <= 4
        L.t2sp_conv2d_direct16_plan(pick(), pick(), pick(), (i32 * 4)(), (ctypes.c_double * 2)())
        L.t2sp_ssyrk_plan(pick(), pick(), rng.choice([64, 128, 256]), (i32 * 3)())
        L.t2sp_ssyrk_workspace_bytes(rng.randint(0, 1), pick(), pick())
        L.t2sp_capsule_direct16_plan(pick(), pick(), (i32 * 6)())
        L.t2sp_mttkrp_workspace_bytes(pick(), pick(), pick(), pick(), 0, 0)
        L.t2sp_capsule_workspace_bytes((i32 * 11)(pick() % 70000 + 1, pick() % 4096 + 1, pick() % 4096 + 1, 7, 7, 3, 3, 2, 4, 4, 4), 0, 0)
        L.t2sp_conv2d_workspace_bytes(pick() % 4096 + 1, pick() % 4096 + 1, pick() % 4096 + 1, pick() % 4096 + 1,
                                      pick() % 4096 + 1, 3, 3)
    assert time.time() - t0 < 60


def _relayout_plan(L, ext, ss, ds):
    nd = len(ext)
    i64 = ctypes.c_int64
    L.t2sp_relayout_plan.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(i64), ctypes.POINTER(i64),
                                     ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
    te, lanes = (ctypes.c_int * nd)(), (ctypes.c_int * 2)()
    took = L.t2sp_relayout_plan(nd, (ctypes.c_int * nd)(*ext), (i64 * nd)(*ss), (i64 * nd)(*ds), te, lanes)
    return took, list(te), list(lanes)


def _strides(ext, order):
    st, s = [0] * len(ext), 1
    for d in order:
        st[d] = s
        s *= ext[d]
    return st


def test_relayout_tiles_cover_the_runs_of_both_sides(lib):
    """The multi-dimensional relayout tile: for the convolution's 10-D tiled output (8 channels, then 7 pixels
    innermost; source rows along the pixels) it is whole along the destination's channel and pixel groups and
    along the source's row, so that 56 of 64 lanes work on both sides; it never exceeds 4096 elements or a
    dimension's extent; plain transposes and tiny boxes go to the other kernels."""
    # cooo, yyy, xxx, coo, yy, xx, y, x, co, n  (fastest first in the destination); source order y.., x.., channels, n
    ext = [8, 7, 1, 1, 2, 2, 4, 28, 32, 16]
    src_order = [1, 4, 6, 2, 5, 7, 0, 3, 8, 9]
    took, te, lanes = _relayout_plan(lib, ext, _strides(ext, src_order), _strides(ext, range(10)))
    assert took == 1
    assert te[0] == 8 and te[1] == 7 and te[4] == 2 and te[6] == 4          # channels x the whole source row of 56
    assert lanes == [56, 56]
    elems = 1
    for t, e in zip(te, ext):
        assert 1 <= t <= e
        elems *= t
    assert 2048 < elems <= 4096
    # a 2-D transpose belongs to the 64 x 64 tile kernel, a box under 4096 elements to the element-wise one
    assert _relayout_plan(lib, [1000, 300], [300, 1], [1, 1000])[0] == 0
    assert _relayout_plan(lib, [8, 7, 5], _strides([8, 7, 5], [1, 2, 0]), _strides([8, 7, 5], [0, 1, 2]))[0] == 0
    # strides that are not positive are not for it
    assert _relayout_plan(lib, [64, 64, 8], [0, 64, 4096], [1, 64, 4096])[0] == 0
    import random
    rng = random.Random(3)
    for _ in range(300):
        nd = rng.randint(2, 8)
        ext = [rng.choice([1, 2, 3, 4, 7, 8, 15, 16, 33, 100, 1000]) for _ in range(nd)]
        so, do = list(range(nd)), list(range(nd))
        rng.shuffle(so)
        rng.shuffle(do)
        took, te, lanes = _relayout_plan(lib, ext, _strides(ext, so), _strides(ext, do))
        if took:
            elems = 1
            for t, e in zip(te, ext):
                assert 1 <= t <= e
                elems *= t
            assert elems <= 4096 and 1 <= lanes[0] <= 64 and 1 <= lanes[1] <= 64


def test_packed_capsule_entry_declines_before_any_launch(lib):
    """t2sp_capsule_packed_f32 checks its operands on the host: sizes that are not positive are errors, strides or
    addresses off the 128-bit grid, a CII that is not a multiple of 4 or does not divide CI, and batches the library
    plans another kernel for (thousands of images: LDS tiles) are declined with 1; nothing is launched in either case,
    so the call is safe without a device."""
    lib.t2sp_set_machine(256, 8)
    i64 = ctypes.c_int64
    f = lib.t2sp_capsule_packed_f32
    f.argtypes = [ctypes.c_void_p, i64, ctypes.c_void_p, i64, ctypes.c_void_p, i64] + [ctypes.c_int] * 5 + [ctypes.c_void_p]
    P, W, V = 0x10000, 0x20000, 0x30000          # never dereferenced on these paths
    ldp, ldw, ldv = 16 * 16 * 32, 4 * 32, 32 * 16 * 16
    assert f(P, ldp, W, ldw, V, ldv, 0, 16, 32, 32, 4, None) == -8
    assert f(P, ldp, W, ldw, V, 0, 2, 16, 32, 32, 4, None) == -8
    assert f(P, ldp + 2, W, ldw, V, ldv, 2, 16, 32, 32, 4, None) == 1
    assert f(P + 4, ldp, W, ldw, V, ldv, 2, 16, 32, 32, 4, None) == 1
    assert f(P, ldp, W, ldw, V, ldv, 2, 16, 32, 32, 6, None) == 1
    assert f(P, ldp, W, ldw, V, ldv, 2, 16, 32, 32, 64, None) == 1
    assert f(P, ldp, W, ldw, V, ldv, 2, 16, 30, 32, 2, None) == 1
    assert f(P, ldp, W, ldw, V, ldv, 256, 16, 32, 32, 4, None) == 1          # 4096 images: rounds of LDS tiles
