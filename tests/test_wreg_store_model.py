"""Host model of how k_gemm_i8_wreg (onnx-mlir_amd/csrc/gemm_wreg.hip) gets its
8-bit results out: every lane writes one byte a K step into a 32 x 384 staging
tile in LDS, and one K loop later the block's 768 lanes read the tile back 16
bytes each and store whole 128-byte lines through a buffer descriptor whose
range check drops what lies past the matrix.  No GPU: the index arithmetic of
the kernel restated for the host, lane by lane, and checked for what the
kernel relies on -- every byte of the staging tile written once and read once,
no lane outside it, every element of the [M, N] result stored exactly once
and nothing stored outside it -- over full, ragged and tiny shapes.  It also
restates the kernel's count of the LDS operations that are younger than an
operand read (its explicit lgkmcnt waits) from the order in which a K step
issues them.
"""
import numpy as np
import pytest

KH, WAVES, NR, PF = 24, 12, 4, 3
PITCH = 32 * WAVES + 16           # kStagePitch
STAGE_BYTES = 32 * PITCH          # kStageBytes
TILE_BYTES = KH * 1024
STAGE_AT = (NR + 1) * TILE_BYTES  # kStageAt
EPI_FIRST, FIX_READ, FIX_WRITE, FLUSH_READ = 2, 12, 16, KH - PF


def block_of(pid, nb, regions_m, regions_n):
    """blockIdx.x -> (row region, column region), as the kernel maps it."""
    per = nb >> 3
    if per > 0 and pid < per * 8:
        pid = (pid & 7) * per + (pid >> 3)
    in_group = 8 * regions_n
    group = pid // in_group
    first_m = group * 8
    gsize = min(regions_m - first_m, 8)
    return first_m + (pid % in_group) % gsize, (pid % in_group) // gsize


def staging_writes():
    """LDS byte offset (from the staging tile's start) of lane (wave, lane),
    accumulator register r: saddr + the instruction's immediate offset."""
    out = {}
    for wave in range(WAVES):
        for lane in range(64):
            l32, lh = lane & 31, lane >> 5
            saddr = 4 * lh * PITCH + wave * 32 + l32
            for r in range(16):
                row = 8 * (r >> 2) + (r & 3)        # + 4 * lh, in saddr
                out[(wave, lane, r)] = saddr + row * PITCH
    return out


def test_staging_tile_is_written_once_and_read_once():
    w = staging_writes()
    offs = np.array(sorted(w.values()))
    assert offs.min() >= 0 and offs.max() < STAGE_BYTES
    assert len(set(w.values())) == len(w) == 32 * 32 * WAVES
    # the byte of result (row, col) of the tile sits at row * PITCH + col
    for (wave, lane, r), off in w.items():
        row = 8 * (r >> 2) + (r & 3) + 4 * (lane >> 5)
        col = wave * 32 + (lane & 31)
        assert off == row * PITCH + col
    # read back: lane idx of the block takes 16 bytes
    read = set()
    for idx in range(WAVES * 64):
        frow, fch = idx // (2 * WAVES), idx % (2 * WAVES)
        base = frow * PITCH + fch * 16
        assert base % 16 == 0 and base + 16 <= STAGE_BYTES
        for b in range(16):
            assert base + b not in read
            read.add(base + b)
    assert read == set(w.values())
    # the two staging tiles lie behind the operand tiles and inside the 160 KB of LDS
    assert STAGE_AT + 2 * STAGE_BYTES <= 160 * 1024


@pytest.mark.parametrize("M,N", [(4096, 3072), (4097, 2304), (129, 512), (300, 896), (1000, 384), (1, 128),
                                 (2945, 3040 // 128 * 128)])
def test_every_result_byte_is_stored_exactly_once(M, N):
    assert N % 128 == 0  # what wreg_ok asks of 8-bit results
    regions_m = (M + 32 * NR - 1) // (32 * NR)
    regions_n = ((N + 31) // 32 + WAVES - 1) // WAVES
    nb = regions_m * regions_n
    assert M * N <= 1 << 31 and 32 * NR * N < 1 << 30
    count = np.zeros(M * N, np.uint8)
    seen = set()
    idx = np.arange(WAVES * 64)
    frow, fch = idx // (2 * WAVES), idx % (2 * WAVES)
    for pid in range(nb):
        rm, rn = block_of(pid, nb, regions_m, regions_n)
        assert (rm, rn) not in seen and rm < regions_m and rn < regions_n
        seen.add((rm, rn))
        row0 = rm * 32 * NR
        for t in range(NR):
            stage_row0 = (row0 + 32 * t) * N            # advanced by 32 * N a tile
            col = rn * 32 * WAVES + fch * 16
            off = np.where(col < N, stage_row0 + frow * N + col, 0x80000000).astype(np.int64)
            assert (off < 1 << 32).all()                # no 32-bit offset wraps
            # the descriptor covers exactly M * N bytes: a 16-byte piece is stored
            # where all of it is in range (N % 16 == 0: none straddles the end)
            inside = off + 16 <= M * N
            assert ((off >= M * N) | inside).all()
            for o in off[inside]:
                count[o:o + 16] += 1
    assert (count == 1).all()


def younger_than_read(s, first, staged, fix):
    """LDS operations issued behind the operand read for step s (issued at the
    top of step s - PF) when step s waits for it, from the order of a K step:
    [fix-up reads at FIX_READ] [fix-up writes at FIX_WRITE] [the gathered
    tile's read at FLUSH_READ] operand read for s + PF, wait, MFMA, [the
    staged byte, steps EPI_FIRST .. EPI_FIRST + 15]."""
    n = 0
    for step in range(s - PF, s + 1):
        st = step % KH
        before_read = []
        if fix and st == FIX_READ:
            before_read += ["fix"] * 2
        if fix and st == FIX_WRITE:
            before_read += ["fix"] * 2
        if staged and not first and st == FLUSH_READ and step >= 0:
            before_read += ["flush"]
        after_wait = []
        if staged and not first and EPI_FIRST <= st < EPI_FIRST + 16 and step >= 0:
            after_wait += ["byte"]
        if step == s - PF:
            n += len(after_wait)                      # behind that step's operand read
        elif step == s:
            n += len(before_read) + 1                 # up to this step's own operand read
        else:
            n += len(before_read) + 1 + len(after_wait)
    return n


def wreg_younger(s, pf, fix_ops, fix_read, fix_write, staged, epi_first, flush_read):
    """The kernel's constexpr of the same name."""
    x = pf
    if fix_read <= s < fix_read + pf:
        x += fix_ops
    if fix_write <= s < fix_write + pf:
        x += fix_ops
    if staged:
        x += sum(1 for j in range(s - pf, s) if epi_first <= j < epi_first + 16)
        if flush_read <= s < flush_read + pf:
            x += 1
    return x


@pytest.mark.parametrize("staged", [False, True])
@pytest.mark.parametrize("fix", [False, True])
def test_lgkm_counts_follow_from_the_order_of_a_step(staged, fix):
    for first in (True, False):
        st = staged and not first
        for s in range(KH):
            if first and s < PF:
                continue  # (the reads of the first steps are issued before the loop)
            want = younger_than_read(s, first, staged, fix)
            got = wreg_younger(s, PF, 2 if fix else 0, FIX_READ, FIX_WRITE, st, EPI_FIRST, FLUSH_READ)
            assert got == want, (staged, fix, first, s, got, want)
            assert got <= 15  # the counter's range


# ---------------------------------------------------------------------------
# vmcnt: "tile t + 1 has landed" = at most Need::at(t) operations outstanding
# ---------------------------------------------------------------------------
CPT, B_FIRST = KH // WAVES, 8


def wreg_need(t, wait_step, staged):
    """The kernel's WregNeed<...>::at(t)."""
    b_late = KH - B_FIRST
    b_seen = b_late if t > 0 else min(wait_step, b_late)
    here = min(wait_step - EPI_FIRST, 16)
    stores = 0 if t == 0 else (t - 1 if staged else 16 * (t - 1) + here)
    return CPT * (NR - 2 - t) + b_seen + stores


def wave_memory_ops(wait_step, staged):
    """A wave's vector-memory operations in program order, as (kind, tile)
    tuples, with ("wait", t) where tile t waits for tile t + 1."""
    ops = [("param", 0)] * 8
    ops += [("copy", 0)] * CPT
    ops += [("b", 0)] * B_FIRST
    for t in range(1, NR):
        ops += [("copy", t)] * CPT
    for t in range(NR):
        for s in range(KH):
            if s == wait_step and t < NR - 1:
                ops.append(("wait", t))
            if t == 0 and s + B_FIRST < KH:
                ops.append(("b", 0))            # behind the step's MFMA
            if t > 0 and not staged and EPI_FIRST <= s < EPI_FIRST + 16:
                ops.append(("store", t - 1))
            if t > 0 and staged and s == KH - 1:
                ops.append(("store", t - 1))
    return ops


@pytest.mark.parametrize("staged", [False, True])
@pytest.mark.parametrize("fix", [False, True])
def test_vmcnt_counts_follow_from_the_order_of_the_loop(staged, fix):
    wait_step = FIX_READ if fix else KH - PF
    ops = wave_memory_ops(wait_step, staged)
    for t in range(NR - 1):
        at = ops.index(("wait", t))
        last_copy = max(i for i, o in enumerate(ops[:at]) if o == ("copy", t + 1))
        younger = sum(1 for o in ops[last_copy + 1:at] if o[0] != "wait")
        assert wreg_need(t, wait_step, staged) == younger, (staged, fix, t)
        assert younger <= 63  # the counter's range
    # the first wait of the kernel, before the loop: tile 0's copies have landed
    # when at most the first loads of Bp and the copies of the other tiles,
    # which were issued behind them, are outstanding
    prologue = 8 + CPT + B_FIRST + CPT * (NR - 1)   # everything issued before the loop
    last_copy0 = max(i for i, o in enumerate(ops[:prologue]) if o == ("copy", 0))
    assert len(ops[last_copy0 + 1:prologue]) == B_FIRST + CPT * (NR - 1)  # the kernel's constant
    assert all(o[0] in ("b", "copy") for o in ops[last_copy0 + 1:prologue])
