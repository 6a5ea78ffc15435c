"""Host model of every global and LDS access of k_gemm_i8_bs as it is shipped
(onnx-mlir_amd/csrc/gemm_kernels.hip, instantiation <TM=4, TN=2, D=4, NST=4,
PIPE>), of its epilogue's stores (gemm_epilogue.h), of k_pad_rows and of the
buffer pool's size arithmetic (runtime.hip), checked against the real extents
of the operands over a grid of shapes; and of the kernel's count of outstanding
memory operations (its explicit vmcnt waits).  No GPU: this is index arithmetic
restated for the host, lane by lane.

Why it exists: a benchmark loop on 4096 x 1040 x 4096 (rows padded to 1088
bytes, 17 K steps, this instantiation) once ended with an illegal memory
access that nothing in the suite shows.  The model finds every access of that
launch in bounds and every wait sufficient (the assertions below hold for it),
so the cause is not in what is modelled here; the padding path stays out of
the library, and the dispatch keeps this kernel to step counts that are
multiples of four (test_dispatch_keeps_bs_to_whole_trips in the GPU suite).
The model of the waits does find the defect of the other development variant
that failed on the device, the one with six LDS stages (see the last tests of
the wait model).
"""
import numpy as np
import pytest

BK = 64


def round_up(a, b):
    return (a + b - 1) // b * b


# ---------------------------------------------------------------------------
# the kernel's block -> tile map (XCD interleave, then groups of 8 row tiles)
# ---------------------------------------------------------------------------
def tile_of(pid, nb, tiles_m, tiles_n):
    per = nb >> 3
    if per > 0 and pid < per * 8:
        pid = (pid & 7) * per + (pid >> 3)
    group_rows = 8
    in_group = group_rows * tiles_n
    group = pid // in_group
    first_m = group * group_rows
    gsize = min(tiles_m - first_m, group_rows)
    tm = first_m + (pid % in_group) % gsize
    tn = (pid % in_group) // gsize
    return tm, tn


@pytest.mark.parametrize("tiles_m,tiles_n", [(32, 16), (33, 16), (1, 1), (7, 3), (8, 43), (17, 5), (64, 1), (3, 100)])
def test_every_tile_is_computed_exactly_once(tiles_m, tiles_n):
    nb = tiles_m * tiles_n
    seen = {tile_of(p, nb, tiles_m, tiles_n) for p in range(nb)}
    assert len(seen) == nb
    assert all(0 <= tm < tiles_m and 0 <= tn < tiles_n for tm, tn in seen)


# ---------------------------------------------------------------------------
# global and LDS addresses
# ---------------------------------------------------------------------------
def lds_off(r, c):
    return r * BK + ((c ^ ((r >> 2) & 3)) << 4)


def check_bs(M, K, N, es, TM=4, TN=2, D=4, NST=4):
    """Every address of one launch; es: bytes of an output element."""
    assert K % BK == 0, "the fast path takes whole K steps only"
    BM, BN = 32 * TM, 4 * 32 * TN
    KT = K // BK
    Npad = round_up(N, 256)
    tiles_m, tiles_n = (M + BM - 1) // BM, (N + BN - 1) // BN
    a_bytes, bp_bytes, out_bytes = M * K, Npad * K, M * N * es
    CA = BM // 64
    STAGE = BM * BK
    lane = np.arange(64)
    l32, lh = lane & 31, lane >> 5
    crow, cchunk = lane >> 2, (lane & 3) ^ ((lane >> 4) & 3)
    # steps the prologue and the loop ask for: 0 .. KT - 1 + max(D, NST - 1),
    # clamped to the last one
    steps = np.minimum(np.arange(KT + max(D, NST - 1)), KT - 1)

    for tm in range(tiles_m):
        m0 = tm * BM
        for wave in range(4):
            for h in range(CA):
                # A copies (global_load_lds, 16 bytes a lane)
                r = (wave * CA + h) * 16 + crow
                rc = np.where(m0 + r < M, r, M - 1 - m0)
                assert (rc >= 0).all() and (m0 + rc < M).all()
                ga = rc * K + cchunk * 16
                assert ga.max() < 2 ** 32
                addr = m0 * K + steps[:, None] * BK + ga[None, :]
                assert addr.min() >= 0 and addr.max() + 16 <= a_bytes, (M, K, N, tm, wave, h)
                # their LDS side: 1 KiB per copy, lane * 16 within it, in a stage
                for stage in range(NST):
                    dst = stage * STAGE + (wave * CA + h) * 1024 + lane * 16
                    assert dst.max() + 16 <= NST * STAGE
                    # the copy puts row r's chunk where the operand reads look for it
                    assert (dst - stage * STAGE == lds_off(r, cchunk)).all()
    # operand reads of A from LDS
    for s2 in range(2):
        for i in range(TM):
            ra = lds_off(l32, s2 * 2 + lh) + i * 2048
            assert ra.max() + 16 <= STAGE

    for tn in range(tiles_n):
        n0 = tn * BN
        for wave in range(4):
            ncol0 = n0 + wave * 32 * TN
            # Bp by buffer loads: descriptor base and range, lane and step offsets
            base = (ncol0 >> 5) * KT * 2048
            records = TN * KT * 2048
            assert base + records <= bp_bytes, (M, K, N, tn, wave)
            for j in range(TN):
                boff = j * KT * 2048 + lane * 16
                for sub in range(2):
                    off = boff[None, :] + steps[:, None] * 2048 + sub * 1024
                    assert off.min() >= 0 and off.max() + 16 <= records
            # the epilogue's per-column operands: clamped to the last column
            for j in range(TN):
                n = ncol0 + j * 32 + l32
                nc = np.where(n < N, n, N - 1)
                assert (nc >= 0).all() and (nc < N).all()

    # the epilogue's stores
    for tm in range(tiles_m):
        for tn in range(tiles_n):
            for wave in range(4):
                mrow0, ncol0 = tm * BM, tn * BN + wave * 32 * TN
                full = (mrow0 + 32 * TM <= M and ncol0 + 32 * TN <= N and
                        N * (32 * TM + 8) * 4 < 2 ** 31)
                if full:
                    # buffer stores: descriptor at the wave tile's first element,
                    # no range check (0x7FFFFFFF records): lane offset + scalar row offset
                    base = (mrow0 * N + ncol0) * es
                    loff = (4 * lh * N + l32) * es
                    worst = 0
                    for i in (0, TM - 1):
                        for r in (0, 15):
                            rowb = (i * 32 + 8 * (r >> 2) + (r & 3)) * N * es
                            for j in (0, TN - 1):
                                voff = loff + j * 32 * es
                                assert voff.max() + rowb < 2 ** 31
                                worst = max(worst, int(base + voff.max() + rowb + es))
                    assert worst <= out_bytes, (M, K, N, tm, tn, wave)
                else:
                    # element by element, each guarded by m < M and n < N
                    m = mrow0 + np.arange(32 * TM)
                    n = ncol0 + np.arange(32 * TN)
                    mm, nn = np.meshgrid(m[m < M], n[n < N], indexing="ij")
                    if mm.size:
                        assert int((mm * N + nn).max() + 1) * es <= out_bytes


SHAPES = [(4096, 1024, 4096), (4096, 1088, 4096),  # 17 steps: the launch that once died
          (2048, 4096, 11008), (4096, 3072, 768), (4100, 1088, 4000), (4096, 64, 4096),
          (4096, 320, 4100), (129, 192, 257), (8192, 11008, 4096), (4095, 2048, 8190)]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("es", [1, 4])
def test_every_access_of_the_shipped_instantiation_is_in_bounds(M, K, N, es):
    check_bs(M, K, N, es)


# ---------------------------------------------------------------------------
# the count of outstanding memory operations
# ---------------------------------------------------------------------------
def wait_counts(TM, TN, D, NST, PIPE):
    CA = (32 * TM) // 64
    PER_STEP = CA + 2 * TN
    AHEAD = 1 if PIPE else 0
    YOUNGER = (NST - 2 - AHEAD) * PER_STEP
    P0 = (NST - 2) * CA + 2 * D * TN
    return CA, PER_STEP, AHEAD, YOUNGER, P0


def static_asserts_hold(TM, TN, D, NST, PIPE):
    """The kernel's compile-time conditions on its wait counts (the last one
    says that step 0 does not use weights that are still on their way: the
    prologue asks for the rows of NST - 1 steps first and for the weights after
    them, and the first wait lets the youngest YOUNGER operations stand)."""
    CA, PER_STEP, AHEAD, YOUNGER, P0 = wait_counts(TM, TN, D, NST, PIPE)
    return (YOUNGER < 64 and P0 < 64 and NST - 2 - AHEAD >= 0 and D >= NST - 2 and
            2 * TN * (D - 1) >= YOUNGER)


def simulate_waits(KT, TM, TN, D=4, NST=4, PIPE=True):
    """A wave's vector memory operations in issue order; they complete in
    order, so `s_waitcnt vmcnt(n)` guarantees all but the youngest n.  Checks
    that what a step reads has landed when it is read, and that no copy
    overwrites a stage that some wave may still read."""
    CA, PER_STEP, AHEAD, YOUNGER, P0 = wait_counts(TM, TN, D, NST, PIPE)
    ops = []  # (kind, step asked for (before clamping), slot)

    def copy_a(step, stage):
        for _ in range(CA):
            ops.append(("a", step, stage))

    def load_b(step, u, sub):
        for _ in range(TN):
            ops.append(("b", step, (u, sub)))

    def landed(n_outstanding):
        return ops[:max(len(ops) - n_outstanding, 0)]

    for p in range(NST - 1):
        copy_a(p, p)
    for u in range(D):
        load_b(u, u, 0)
        load_b(u, u, 1)
    if PIPE:
        done = landed(P0)
        assert [o for o in done if o[0] == "a" and o[1] == 0] == [("a", 0, 0)] * CA
    stage = 0
    for kt in range(KT):
        u = kt % D
        done = landed(YOUNGER)
        # the stage(s) this step reads hold the step's rows and have landed
        for ahead in range(AHEAD + 1):
            want, st = kt + ahead, (stage + ahead) % NST
            last = [o for o in ops if o[0] == "a" and o[2] == st][-CA:]
            if want < KT:
                assert all(o[1] == want for o in last), (KT, kt, ahead, last)
                idx = max(i for i, o in enumerate(ops) if o[0] == "a" and o[2] == st)
                assert idx < len(done), ("copy not waited for", KT, kt, ahead)
        # this step's weights (both halves) were asked for D steps ago and have landed
        for sub in range(2):
            idx = max(i for i, o in enumerate(ops) if o[0] == "b" and o[2] == (u, sub))
            assert ops[idx][1] == kt and idx < len(done), ("weights", KT, kt, sub)
        load_b(kt + D, u, 0)
        load_b(kt + D, u, 1)
        # refill the stage that was read in the previous step: every wave has
        # passed this step's barrier, after it finished those reads
        target = (stage - 1) % NST
        assert target not in [(stage + a) % NST for a in range(AHEAD + 1)]
        copy_a(kt + NST - 1, target)
        stage = (stage + 1) % NST


def model_accepts(TM, TN, D, NST, PIPE):
    try:
        for KT in list(range(1, 24)) + [64, 172]:
            simulate_waits(KT, TM, TN, D=D, NST=NST, PIPE=PIPE)
    except AssertionError:
        return False
    return True


def test_shipped_instantiation_waits_for_what_each_step_reads():
    for KT in list(range(1, 40)) + [64, 172]:
        simulate_waits(KT, 4, 2, D=4, NST=4, PIPE=True)
    assert static_asserts_hold(4, 2, 4, 4, True)


@pytest.mark.parametrize("NST,D", [(3, 4), (4, 4), (4, 2), (4, 3), (5, 4), (6, 4), (6, 6), (6, 8)])
def test_compile_time_conditions_reject_what_the_model_rejects(NST, D):
    """For every tile shape and depth: an instantiation passes the kernel's
    static_asserts only if the model finds its waits sufficient."""
    for PIPE in (True, False):
        if NST - 2 - (1 if PIPE else 0) < 0:
            continue
        for TM in (2, 4):
            for TN in (1, 2, 3, 4):
                if static_asserts_hold(TM, TN, D, NST, PIPE):
                    assert model_accepts(TM, TN, D, NST, PIPE), (TM, TN, D, NST, PIPE)


def test_six_stage_variant_used_weights_that_had_not_landed():
    """The development instantiation with six LDS stages (64 x 128 tiles: TM =
    2, TN = 1, D = 4) that ended in a fault or hang on the device: its first
    wait lets nine operations stand, and the eight loads of the weights come
    after the rows in the prologue, so step 0 multiplied with registers whose
    loads were still in flight.  The kernel now refuses to compile so."""
    assert not model_accepts(2, 1, 4, 6, True)
    assert not static_asserts_hold(2, 1, 4, 6, True)


# ---------------------------------------------------------------------------
# k_pad_rows and the pool
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("M,K", [(1, 1), (16, 4100), (64, 1001), (33, 15), (64, 65537), (5, 16)])
def test_pad_rows_stays_inside_both_buffers(M, K):
    Kp = round_up(K, 16)
    assert 1 <= M <= 64
    grid_x = (Kp + 1023) // 1024
    out_bytes = M * Kp  # what the runtime asks the pool for
    hi_in = hi_out = 0
    for r in (0, M - 1):
        for bx in range(grid_x):
            c = bx * 256 + np.arange(256)
            while c.min() < Kp:
                cc = c[c < Kp]
                hi_out = max(hi_out, int(r * Kp + cc.max()) + 1)
                rd = cc[cc < K]
                if rd.size:
                    hi_in = max(hi_in, int(r * K + rd.max()) + 1)
                c = c + grid_x * 256
    assert hi_in <= M * K and hi_out <= out_bytes
    assert hi_out == out_bytes  # and every byte of the padded rows is written


def test_pool_blocks_are_never_smaller_than_asked_for():
    """Ctx::take: the request rounded up to 256 bytes; an idle block serves it
    if it is the smallest one that is large enough and at most twice as large."""
    rng = np.random.default_rng(0)
    pool = []  # capacities of idle blocks
    for _ in range(2000):
        want = int(rng.integers(0, 1 << 24))
        need = round_up(max(want, 16) if want else 16, 256)
        fits = sorted(c for c in pool if c >= need)
        if fits and fits[0] <= 2 * need:
            cap = fits[0]
            pool.remove(cap)
        else:
            cap = need
        assert cap >= want and cap >= need
        if rng.integers(0, 2):
            pool.append(cap)
    # the sizes of the launch that died: 4096 rows of 1088 bytes, and its packed weights
    for want in (4096 * 1088, 1088 * 4096, 4096 * 4096 * 4):
        assert round_up(want, 256) >= want
