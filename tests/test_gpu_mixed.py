"""All bit-width groups of a bucket in one launch (dq_mixed_*), against the per-group calls they replace
(testbed_evaluation/new_comm_hooks/comm_hooks.py:963-1018 runs the ring once per group) and against the
oracle -- byte for byte."""
import numpy as np
import pytest
import torch

from helpers import BF16, F32, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REC = {8: 274, 4: 146, 2: 82}


def bits_t(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def make_plan(capi, nsc, seed, weights=(1, 1, 1)):
    g = torch.Generator().manual_seed(seed)
    w = torch.tensor(weights, dtype=torch.float)
    q = torch.tensor([8, 4, 2])[torch.multinomial(w, nsc, replacement=True, generator=g)].to(DEV)
    order = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    capi.group_plan(q, order, work)
    return q, order, work


def segments(counts, chunk, world, nsc):
    """(width, entry of `order` where the run's rows start, row of the random pool of its first record, records, byte
    offset) of ring chunk `chunk`, and the stream size"""
    out, pos, off = [], 0, 0
    for g, (q, n) in enumerate(zip((8, 4, 2), counts)):
        per = -(-n // world)
        begin = min(per * chunk, n)
        cnt = min(per, n - begin)
        out.append((q, g * nsc + begin, pos + begin, cnt, off))
        pos += n
        off += cnt * REC[q]
    return out, off


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("strategy", [2, 3])
@pytest.mark.parametrize("nsc,world,weights", [(1037, 1, (1, 1, 1)), (1037, 3, (1, 2, 3)), (2, 1, (1, 1, 1)),
                                               (515, 4, (1, 0, 1)), (64, 8, (0, 1, 0)), (6403, 8, (1, 6, 2)),
                                               (2051, 7, (1, 3, 1)), (4099, 13, (2, 5, 1))])
def test_mixed_matches_per_group_calls(capi, dt, strategy, nsc, world, weights):
    n_valid = nsc * 256 - 77
    q, order, work = make_plan(capi, nsc, nsc + world, weights)
    counts = work[:3].tolist()
    assert sum(counts) == nsc
    g = torch.Generator().manual_seed(nsc * 3 + strategy)
    full = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
    peer = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
    stats = torch.randn(nsc, 2, generator=g).mul(1e-2).to(torch.bfloat16).to(DEV)
    pool = torch.rand(nsc * 256, generator=g).to(torch.bfloat16 if (dt == torch.bfloat16 or strategy == 2) else dt).to(DEV)
    cap = capi.mixed_required_bytes(nsc, world)
    out = torch.full((n_valid + 300,), 7.0, dtype=dt, device=DEV)
    out_ref = torch.full((n_valid + 300,), 7.0, dtype=dt, device=DEV)
    for chunk in range(world):
        segs, total = segments(counts, chunk, world, nsc)
        assert total <= cap
        enc = torch.full((cap + 16,), 0xAB, dtype=torch.uint8, device=DEV)
        send = torch.full((cap + 16,), 0xCD, dtype=torch.uint8, device=DEV)
        capi.mixed_compress(full, order, work, enc, nsc, strategy, rand_pool=pool, ring_chunk=chunk, ring_world=world)
        peer_before = peer.clone()
        capi.mixed_compress(peer, order, work, send, nsc, strategy, rand_pool=pool, recv=enc, ring_chunk=chunk,
                            ring_world=world)
        assert torch.equal(peer, peer_before)
        capi.mixed_decompress(send, out, order, work, nsc, strategy, stats=stats, n_limit=n_valid, ring_chunk=chunk,
                              ring_world=world)
        assert bool((enc[total:] == 0xAB).all()) and bool((send[total:] == 0xCD).all())    # nothing past the stream
        for width, row0, pos, cnt, off in segs:
            if cnt == 0:
                continue
            rows = order[row0:row0 + cnt]
            rnd = pool[pos * 256:(pos + cnt) * 256]
            nb = cnt * REC[width]
            e = torch.zeros(nb, dtype=torch.uint8, device=DEV)
            s = torch.zeros(nb, dtype=torch.uint8, device=DEV)
            capi.scaling_compress_rows(full, rows, e, rnd, cnt, width, strategy)
            capi.scaling_dec_comp_rows(e, peer, rows, s, rnd, cnt, width, strategy)
            assert torch.equal(enc[off:off + nb], e), (chunk, width)
            assert torch.equal(send[off:off + nb], s), (chunk, width)
            capi.scaling_decompress_rows(s, out_ref, rows, stats, n_valid, cnt, width, strategy)
    assert torch.equal(bits_t(out), bits_t(out_ref))
    assert bool((out[n_valid:] == 7.0).all())


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("strategy,world", [(2, 1), (3, 2)])
def test_long_runs_take_the_decoders_of_several_tiles_per_wave(capi, dt, strategy, world):
    """From 262,144 superchunks per ring chunk (or rows of a list) on, the decoders run as waves of four tiles that fetch
    their row-list entries with one load.  Their output must be that of the one-tile kernels, which the same records
    reach here in pieces of 100,000 rows."""
    nsc = 450_001 * world + 5
    n_valid = nsc * 256 - 77
    q, order, work = make_plan(capi, nsc, 11 + world, (1, 6, 2))
    counts = work[:3].tolist()
    g = torch.Generator(device=DEV).manual_seed(5 + strategy)
    full = (torch.randn(nsc * 256, generator=g, device=DEV) * 1e-2).to(dt)
    stats = torch.randn(nsc, 2, generator=g, device=DEV).mul(1e-2).to(torch.bfloat16)
    cap = capi.mixed_required_bytes(nsc, world)
    out = torch.full((n_valid + 300,), 7.0, dtype=dt, device=DEV)
    out_ref = torch.full((n_valid + 300,), 7.0, dtype=dt, device=DEV)
    out_rows = torch.full((n_valid + 300,), 7.0, dtype=dt, device=DEV)
    long_runs = 0
    for chunk in range(world):
        segs, total = segments(counts, chunk, world, nsc)
        enc = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        capi.mixed_compress(full, order, work, enc, nsc, strategy, seed=3, step=chunk, ring_chunk=chunk, ring_world=world)
        capi.mixed_decompress(enc, out, order, work, nsc, strategy, stats=stats, n_limit=n_valid, ring_chunk=chunk,
                              ring_world=world)
        for width, row0, pos, cnt, off in segs:
            rows = order[row0:row0 + cnt]
            for a in range(0, cnt, 100_000):
                b = min(cnt, a + 100_000)
                capi.scaling_decompress_rows(enc[off + a * REC[width]:off + b * REC[width]], out_ref, rows[a:b], stats, n_valid,
                                             b - a, width, strategy)
            capi.scaling_decompress_rows(enc[off:off + cnt * REC[width]], out_rows, rows, stats, n_valid, cnt, width, strategy)
            long_runs += cnt >= 262144
    assert long_runs >= 1                  # the row-list decoder took its long variant as well
    assert torch.equal(bits_t(out), bits_t(out_ref))
    assert torch.equal(bits_t(out_rows), bits_t(out_ref))
    assert bool((out[n_valid:] == 7.0).all()) and bool((out_rows[n_valid:] == 7.0).all())
    # and the decoded values are the source to within the 2-bit step of its widest class
    assert float((out[:n_valid].float() - stats[:, 0].float().repeat_interleave(256)[:n_valid] - full[:n_valid].float()).abs().max()) < 0.1


@pytest.mark.parametrize("dt,odt", [(torch.bfloat16, BF16), (torch.float32, F32)])
@pytest.mark.parametrize("strategy", [2, 3])
def test_mixed_philox_matches_oracle(capi, oracle, dt, odt, strategy):
    """in-kernel rounding stream keyed by the chunk's index in the source vector: every run equals the oracle's
    compress of the gathered superchunks with the gathered uniform values"""
    nsc, seed, step = 333, 2027, 5
    q, order, work = make_plan(capi, nsc, 17)
    counts = work[:3].tolist()
    g = torch.Generator().manual_seed(5)
    full = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
    enc = torch.zeros(capi.mixed_required_bytes(nsc, 1), dtype=torch.uint8, device=DEV)
    capi.mixed_compress(full, order, work, enc, nsc, strategy, seed=seed, step=step)
    uni = oracle.philox_uniform(nsc * 256, seed, step)
    if odt == BF16:
        uni = (uni.view(np.uint32) >> 16).astype(np.uint16)     # k/256 is exact in bf16
    src_h = to_bits(full.cpu())
    ord_h = order.cpu().numpy()
    segs, total = segments(counts, 0, 1, nsc)
    got = enc.cpu().numpy()
    for width, row0, pos, cnt, off in segs:
        rows = ord_h[row0:row0 + cnt]
        gs = src_h.reshape(-1, 256)[rows].reshape(-1).copy()
        gu = uni.reshape(-1, 256)[rows].reshape(-1).copy()
        want = oracle.scaling_compress(gs, gu, cnt * 256, width, 16, strategy, odt)
        assert (got[off:off + cnt * REC[width]] == want).all(), width
    # natural order (rows == identity) of the single-width Philox call uses the same key
    e4 = torch.zeros(capi.required_bytes(nsc * 256, 4, 16, strategy), dtype=torch.uint8, device=DEV)
    capi.scaling_compress_philox(full, e4, nsc * 256, 4, 16, strategy, seed, step)
    want = oracle.scaling_compress(src_h, uni, nsc * 256, 4, 16, strategy, odt)
    assert (e4.cpu().numpy() == want).all()


@pytest.mark.parametrize("dt,odt", [(torch.bfloat16, BF16), (torch.float32, F32)])
@pytest.mark.parametrize("world", [1, 2, 3, 8, 6, 24])
@pytest.mark.parametrize("n", [256 * 40, 256 * 41 - 200, 256 * 41 - 1, 77])
def test_stats_and_centre_on_load(capi, oracle, dt, odt, world, n):
    """superchunk_stats == the oracle's statistics and binary32 means; compress with the centring folded into the
    load == mean_center followed by compress of the residual, with nothing read beyond n"""
    nsc = (n + 255) // 256
    g = torch.Generator().manual_seed(n + world)
    base = torch.randn(n, generator=g) * 1e-2 + 3e-3
    if n >= 1024:
        # superchunks at the bottom of the exponent range: element / world is a denormal binary32 number there, and
        # the centred value must still be the one of the two-step arithmetic
        base[256:512] = torch.randn(256, generator=g) * 1e-39
        base[512:768] = torch.randn(256, generator=g) * 3e-38
        # element / world exactly half-way between two subnormal numbers (m 2^-150, m odd; representable in binary32 for
        # an even world size that is not a power of two), in pairs that cancel in the first step of the mean's tree:
        # the mean is zero and the residual is the rounded quotient itself
        m = torch.randint(0, 500, (128,), generator=g).double() * 2 + 1
        tie = m * world * 2.0 ** -150
        base = base.double()
        base[768:896] = tie
        base[896:1024] = -tie
        base = base.float()
    src = torch.full((n + 64,), float("nan"), dtype=dt, device=DEV)     # a NaN beyond n must never be picked up
    src[:n] = base.to(dt)
    stats = torch.zeros(nsc, 2, dtype=torch.bfloat16, device=DEV)
    mean = torch.zeros(nsc, dtype=torch.float32, device=DEV)
    capi.superchunk_stats(src, stats, mean, n, world)
    st_o, mean_o = oracle.superchunk_stats(to_bits(src[:n].cpu()), n, world, odt)
    assert (to_bits(stats.cpu()).reshape(-1) == st_o).all()
    assert (mean.cpu().numpy().view(np.uint32) == mean_o.view(np.uint32)).all()
    stats2 = torch.zeros_like(stats)
    capi.superchunk_stats(src, stats2, None, n, world)
    assert torch.equal(bits_t(stats), bits_t(stats2))

    residual = torch.zeros(nsc * 256, dtype=dt, device=DEV)
    stats3 = torch.zeros_like(stats)
    capi.superchunk_mean_center(src, residual, stats3, n, world)
    assert torch.equal(bits_t(stats), bits_t(stats3))
    res_o, _ = oracle.superchunk_mean_center(to_bits(src[:n].cpu()), n, world, odt)
    assert (to_bits(residual.cpu()).view(res_o.dtype if odt != F32 else np.uint32) ==
            (res_o if odt != F32 else res_o.view(np.uint32))).all()
    q, order, work = make_plan(capi, nsc, n)
    pool = torch.rand(nsc * 256, generator=g)
    pool[768:1024] = 0.0        # (a random value of 0 turns the lowest bit of a tiny quotient into a code)
    pool = pool.to(dt).to(DEV)
    cap = capi.mixed_required_bytes(nsc, 1)
    for strategy in (2, 3):
        a = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        b = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        capi.mixed_compress(residual, order, work, a, nsc, strategy, rand_pool=pool)
        capi.mixed_compress(src, order, work, b, nsc, strategy, rand_pool=pool, center_mean=mean, center_world=world, n=n)
        assert torch.equal(a, b), strategy
        # the fused step centres its local operand the same way
        a2, b2 = torch.zeros_like(a), torch.zeros_like(a)
        capi.mixed_compress(residual, order, work, a2, nsc, strategy, seed=9, step=1, recv=a)
        capi.mixed_compress(src, order, work, b2, nsc, strategy, seed=9, step=1, recv=a, center_mean=mean,
                            center_world=world, n=n)
        assert torch.equal(a2, b2), strategy


def test_mixed_misaligned_buffers(capi):
    """element buffers that are only element-aligned and streams at odd byte offsets"""
    nsc = 203
    q, order, work = make_plan(capi, nsc, 3)
    g = torch.Generator().manual_seed(1)
    dt = torch.bfloat16
    full_al = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
    pool_al = torch.rand(nsc * 256, generator=g).to(dt).to(DEV)
    full = torch.zeros(nsc * 256 + 8, dtype=dt, device=DEV)[3:3 + nsc * 256].copy_(full_al)
    pool = torch.zeros(nsc * 256 + 8, dtype=dt, device=DEV)[1:1 + nsc * 256].copy_(pool_al)
    cap = capi.mixed_required_bytes(nsc, 1)
    ref = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    capi.mixed_compress(full_al, order, work, ref, nsc, 2, rand_pool=pool_al)
    enc = torch.zeros(cap + 16, dtype=torch.uint8, device=DEV)[5:5 + cap]
    capi.mixed_compress(full, order, work, enc, nsc, 2, rand_pool=pool)
    assert torch.equal(enc, ref)
    out_ref = torch.zeros(nsc * 256, dtype=dt, device=DEV)
    capi.mixed_decompress(ref, out_ref, order, work, nsc, 2)
    out = torch.zeros(nsc * 256 + 8, dtype=dt, device=DEV)[1:1 + nsc * 256]
    capi.mixed_decompress(enc, out, order, work, nsc, 2)
    assert torch.equal(bits_t(out), bits_t(out_ref))


def test_mixed_pipeline_replays_as_graph(capi):
    """stats -> plan -> compress -> decompress of a bucket is a fixed launch sequence with no read-back: captured
    once, replayed on new data, every replay equals the eager result"""
    n = 6553600 // 4
    nsc = n // 256
    g = torch.Generator().manual_seed(11)
    scales = torch.exp(torch.randn(nsc, 1, generator=g) * 6.0) * 1e-3
    src = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    stats = torch.zeros(nsc, 2, dtype=torch.bfloat16, device=DEV)
    mean = torch.zeros(nsc, dtype=torch.float32, device=DEV)
    order = torch.zeros(3 * nsc, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    enc = torch.zeros(capi.mixed_required_bytes(nsc, 1), dtype=torch.uint8, device=DEV)
    out = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    u = 7.1

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        src.copy_((torch.randn(nsc, 256, generator=gg) * scales).reshape(-1).to(torch.bfloat16))

    def pipeline(stream=None):
        capi.superchunk_stats(src, stats, mean, n, 1, stream=stream)
        capi.group_plan_stats(stats, u, None, order, work, stream=stream)
        capi.mixed_compress(src, order, work, enc, nsc, 2, seed=1, step=0, center_mean=mean, center_world=1, n=n,
                            stream=stream)
        capi.mixed_decompress(enc, out, order, work, nsc, 2, stats=stats, n_limit=n, stream=stream)

    fill(0)
    pipeline()
    torch.cuda.synchronize()
    counts0 = work[:3].tolist()
    assert min(counts0) > 0, counts0
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            pipeline(side.cuda_stream)
    for seed in (1, 2, 3):
        fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got, got_enc, got_counts = out.clone(), enc.clone(), work[:3].tolist()
        out.zero_()
        pipeline()
        torch.cuda.synchronize()
        assert got_counts == work[:3].tolist()
        total = sum(c * REC[w] for c, w in zip(got_counts, (8, 4, 2)))
        assert torch.equal(got_enc[:total], enc[:total])
        assert torch.equal(bits_t(got), bits_t(out))
        err = (out.float() - src.float()).pow(2).sum() / src.float().pow(2).sum()
        assert float(err) < 0.05


@pytest.mark.parametrize("W", [1, 2, 3])
@pytest.mark.parametrize("strategy", [2, 3])
def test_single_pass_pipeline_matches_oracle(capi, oracle, W, strategy):
    """the whole device-resident all-reduce (statistics, widths, partition, ring of mixed launches, mean add) against
    the oracle's functions chained on the host, bit for bit, for every simulated rank"""
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import dynamic_bitrate_allreduce_single_pass
    n, seed, u = 256 * 301 - 100, 77, 6.0
    nsc = (n + 255) // 256
    g = torch.Generator().manual_seed(W * 10 + strategy)
    scales = torch.exp(torch.randn(nsc, 1, generator=g) * 6.0) * 1e-3
    vecs = [((torch.randn(nsc, 256, generator=g) * scales).reshape(-1)[:n] + 1e-4).to(torch.bfloat16) for _ in range(W)]
    outs, total, counts = dynamic_bitrate_allreduce_single_pass([v.to(DEV) for v in vecs], u, strategy=strategy, seed=seed)
    torch.cuda.synchronize()

    # host chain
    res, stats = [], []
    for v in vecs:
        r, s = oracle.superchunk_mean_center(to_bits(v), n, W, BF16)
        res.append(r.reshape(-1, 256))
        stats.append(torch.from_numpy(s.view(np.int16).copy()).view(torch.bfloat16))
    tot = stats[0].clone()
    for s in stats[1:]:
        tot.add_(s)                                   # bf16 adds, the order of the pipeline
    tot_bits = to_bits(tot)
    assert (to_bits(total.cpu()).reshape(-1) == tot_bits).all()
    qb = oracle.dynamic_bitrate_qbits(tot_bits[1::2].copy(), u)
    cnt = [int((qb == w).sum()) for w in (8, 4, 2)]
    assert counts.tolist() == cnt + [0] and min(cnt) > 0, (counts.tolist(), cnt)
    uni = {}

    def U(rank, step, rows):
        if (rank, step) not in uni:
            x = oracle.philox_uniform(nsc * 256, seed + rank, step)
            uni[(rank, step)] = (x.view(np.uint32) >> 16).astype(np.uint16).reshape(-1, 256)
        return uni[(rank, step)][rows].reshape(-1).copy()

    want = np.zeros((nsc, 256), np.uint16)
    for width in (8, 4, 2):
        rows_g = np.nonzero(qb == width)[0]
        per = -(-rows_g.size // W)
        for c in range(W):
            rows = rows_g[per * c:per * (c + 1)]
            if rows.size == 0:
                continue
            m = rows.size * 256
            stream = oracle.scaling_compress(res[c][rows].reshape(-1).copy(), U(c, 0, rows), m, width, 16, strategy, BF16)
            for s in range(1, W):
                rank = (c + s) % W
                stream = oracle.scaling_dec_comp(stream, res[rank][rows].reshape(-1).copy(), U(rank, s, rows), m, width, 16,
                                                 strategy, BF16)
            dec = np.zeros(m, np.uint16)
            oracle.scaling_decompress(stream, dec, m, width, 16, strategy, BF16)
            want[rows] = dec.reshape(-1, 256)
    final = oracle.superchunk_add_mean_copy(want.reshape(-1), tot_bits, n, BF16)
    for r in range(W):
        assert (to_bits(outs[r].cpu()) == final).all(), r
    exact = torch.stack([v.double() for v in vecs]).sum(0) / W
    err = float((outs[0].cpu().double() - exact).pow(2).sum() / exact.pow(2).sum())
    assert err < 0.02, err


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("strategy", [2, 3])
def test_mixed_special_values(capi, dt, strategy):
    """NaN, infinities, huge, tiny and all-zero superchunks take the guarded path of a wave: the folded calls still equal
    mean_center + the per-width calls, and the random pool may hold values outside [0, 1]"""
    nsc, n = 97, 97 * 256 - 13
    g = torch.Generator().manual_seed(7 + strategy)
    x = torch.randn(n, generator=g) * 1e-2
    x[5] = float("nan"); x[300] = float("inf"); x[301] = float("-inf"); x[1000] = 3e38; x[1001] = -1e-40
    x[256 * 10:256 * 12] = 0.0
    x[256 * 20:256 * 21] = 1e30
    x[256 * 30:256 * 31] = 1e-38
    src = x.to(dt).to(DEV)
    pool = torch.rand(nsc * 256, generator=g)
    pool[77] = 1.5; pool[78] = -0.25; pool[79] = float("nan")
    pool = pool.to(dt).to(DEV)
    q, order, work = make_plan(capi, nsc, 5)
    counts = work[:3].tolist()
    stats = torch.zeros(nsc, 2, dtype=torch.bfloat16, device=DEV)
    mean = torch.zeros(nsc, device=DEV)
    capi.superchunk_stats(src, stats, mean, n, 3)
    residual = torch.zeros(nsc * 256, dtype=dt, device=DEV)
    stats2 = torch.zeros_like(stats)
    capi.superchunk_mean_center(src, residual, stats2, n, 3)
    assert torch.equal(bits_t(stats), bits_t(stats2))
    cap = capi.mixed_required_bytes(nsc, 1)
    enc = torch.zeros(cap, dtype=torch.uint8, device=DEV)
    capi.mixed_compress(src, order, work, enc, nsc, strategy, rand_pool=pool, center_mean=mean, center_world=3, n=n)
    out = torch.full((n,), 7.0, dtype=dt, device=DEV)
    capi.mixed_decompress(enc, out, order, work, nsc, strategy, stats=stats, n_limit=n)
    out_ref = torch.full((n,), 7.0, dtype=dt, device=DEV)
    segs, total = segments(counts, 0, 1, nsc)
    for width, row0, pos, cnt, off in segs:
        rows = order[row0:row0 + cnt]
        e = torch.zeros(cnt * REC[width], dtype=torch.uint8, device=DEV)
        capi.scaling_compress_rows(residual, rows, e, pool[pos * 256:(pos + cnt) * 256], cnt, width, strategy)
        assert torch.equal(enc[off:off + e.numel()], e), width
        capi.scaling_decompress_rows(e, out_ref, rows, stats, n, cnt, width, strategy)
    assert torch.equal(bits_t(out), bits_t(out_ref))


@pytest.mark.parametrize("block", range(6))
def test_mixed_random_shapes(capi, block):
    """seeded random plans, ring splits, element types, random sources and alignments: the one-launch calls against
    the per-width calls on every run of every ring chunk"""
    rng = np.random.default_rng(1000 + block)
    for case in range(12):
        nsc = int(rng.choice([1, 3, 4, 5, 63, 64, 65, 257, 1023, 1500, 4097]))
        world = int(rng.choice([1, 2, 3, 5, 8]))
        weights = tuple(float(w) for w in rng.choice([0.0, 0.2, 1.0, 3.0], size=3))
        if sum(weights) == 0:
            weights = (1.0, 1.0, 1.0)
        dt = [torch.bfloat16, torch.float32][int(rng.integers(2))]
        strategy = int(rng.choice([2, 3]))
        use_philox = bool(rng.integers(2))
        seed = int(rng.integers(1 << 30))
        q, order, work = make_plan(capi, nsc, seed, weights)
        counts = work[:3].tolist()
        g = torch.Generator().manual_seed(seed)
        shift = int(rng.integers(0, 4)) * (8 if dt == torch.bfloat16 else 4) + int(rng.integers(2))   # element offset of the view
        full = torch.zeros(nsc * 256 + 64, dtype=dt, device=DEV)[shift:shift + nsc * 256]
        full.copy_((torch.randn(nsc * 256, generator=g) * float(10.0 ** rng.uniform(-6, 2))).to(dt))
        peer = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
        pool_dt = dt if (dt == torch.bfloat16 or rng.integers(2)) else torch.bfloat16
        pool = torch.rand(nsc * 256, generator=g).to(pool_dt).to(DEV)
        cap = capi.mixed_required_bytes(nsc, world)
        off0 = int(rng.integers(0, 16))
        tag = (block, case, nsc, world, weights, dt, strategy, use_philox, shift, off0)
        for chunk in range(world):
            enc = torch.zeros(cap + 32, dtype=torch.uint8, device=DEV)[off0:off0 + cap]
            send = torch.zeros(cap + 32, dtype=torch.uint8, device=DEV)[off0:off0 + cap]
            kw = dict(seed=seed, step=chunk) if use_philox else dict(rand_pool=pool)
            capi.mixed_compress(full, order, work, enc, nsc, strategy, ring_chunk=chunk, ring_world=world, **kw)
            capi.mixed_compress(peer, order, work, send, nsc, strategy, recv=enc, ring_chunk=chunk, ring_world=world, **kw)
            segs, total = segments(counts, chunk, world, nsc)
            for width, row0, pos, cnt, off in segs:
                if cnt == 0:
                    continue
                rows = order[row0:row0 + cnt]
                nb = cnt * REC[width]
                if use_philox:
                    uni = torch.empty(nsc * 256, dtype=dt, device=DEV)
                    capi.philox_uniform(uni, seed, chunk)
                    rnd = uni.view(-1, 256)[rows.long()].reshape(-1).contiguous()
                else:
                    rnd = pool[pos * 256:(pos + cnt) * 256]
                e = torch.zeros(nb, dtype=torch.uint8, device=DEV)
                s = torch.zeros(nb, dtype=torch.uint8, device=DEV)
                capi.scaling_compress_rows(full, rows, e, rnd, cnt, width, strategy)
                capi.scaling_dec_comp_rows(e, peer, rows, s, rnd, cnt, width, strategy)
                assert torch.equal(enc[off:off + nb], e), tag + (chunk, width)
                assert torch.equal(send[off:off + nb], s), tag + (chunk, width)


def _llama_like(n, seed, dt=torch.bfloat16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    nsc = (n + 255) // 256
    scales = torch.exp(torch.randn(nsc, 1, generator=g, device=DEV) * 6.0) * 1e-3
    return ((torch.randn(nsc, 256, generator=g, device=DEV) * scales).reshape(-1)[:n] + 1e-4).to(dt)


def _four_calls(capi, x, n, u, strategy, seed, step, world=1):
    nsc = (n + 255) // 256
    stats = torch.zeros((nsc, 2), dtype=torch.bfloat16, device=DEV)
    mean = torch.zeros(nsc, dtype=torch.float32, device=DEV)
    order = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    packed = torch.zeros(capi.mixed_required_bytes(nsc, 1), dtype=torch.uint8, device=DEV)
    out = torch.zeros_like(x)
    capi.superchunk_stats(x, stats, mean, n, world)
    capi.group_plan_stats(stats, u, None, order, work)
    capi.mixed_compress(x, order, work, packed, nsc, strategy, seed=seed, step=step, center_mean=mean, center_world=world, n=n)
    capi.mixed_decompress(packed, out, order, work, nsc, strategy, stats=stats, n_limit=n)
    return stats, mean, order, work, packed, out


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("strategy", [2, 3])
def test_bucket_call_equals_the_four_calls(capi, eden_utils, dt, strategy):
    """dq_dynamic_bitrate_bucket enqueues statistics -> plan -> mixed compress -> mixed decompress with one host call: every
    buffer it writes equals what the four calls write, for all stages at once, for the stages one by one, with u in
    device memory, through ctypes and through the module; step_dev adds to the step of the rounding stream"""
    n, u, seed, step = 256 * 700 - 131, 6.0, 11, 5
    nsc = (n + 255) // 256
    x = _llama_like(n, 3, dt)
    ref = _four_calls(capi, x, n, u, strategy, seed, step)
    assert min(ref[3][:3].tolist()) > 0

    def fresh():
        return (torch.zeros((nsc, 2), dtype=torch.bfloat16, device=DEV), torch.zeros(nsc, dtype=torch.float32, device=DEV),
                torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV),
                torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV),
                torch.zeros(capi.mixed_required_bytes(nsc, 1), dtype=torch.uint8, device=DEV), torch.zeros_like(x))

    def same(got):
        counts = ref[3][:3].tolist()
        used = sum(c * r for c, r in zip(counts, (274, 146, 82)))
        assert torch.equal(bits_t(got[0]), bits_t(ref[0])) and torch.equal(bits_t(got[1]), bits_t(ref[1]))
        assert got[3][:4].tolist() == ref[3][:4].tolist()
        for g_, c in enumerate(counts):
            assert torch.equal(got[2][g_ * nsc:g_ * nsc + c], ref[2][g_ * nsc:g_ * nsc + c])
        assert torch.equal(got[4][:used], ref[4][:used])
        assert torch.equal(bits_t(got[5]), bits_t(ref[5]))

    # all stages, u a number
    bufs = fresh()
    desc, dev = capi.bucket_descriptor(x, n, *bufs[:5], strategy=strategy, out=bufs[5], u=u, seed=seed, step=step)
    capi.dynamic_bitrate_bucket(desc, dev)
    same(bufs)
    # stage by stage, u and the step offset in device memory
    bufs = fresh()
    u_dev = torch.full((1,), u, dtype=torch.float64, device=DEV)
    step_dev = torch.full((1,), 3, dtype=torch.int64, device=DEV)
    desc, dev = capi.bucket_descriptor(x, n, *bufs[:5], strategy=strategy, out=bufs[5], u=u_dev, seed=seed, step=step - 3,
                                       step_dev=step_dev)
    for stage in (capi.STAGE_STATS, capi.STAGE_PLAN, capi.STAGE_COMPRESS, capi.STAGE_DECOMPRESS):
        capi.dynamic_bitrate_bucket(desc, dev, stages=stage)
    same(bufs)
    # another value of the device-side step: other random values, other bytes
    step_dev.fill_(4)
    capi.dynamic_bitrate_bucket(desc, dev, stages=capi.STAGE_COMPRESS)
    assert not torch.equal(bufs[4], ref[4])
    # the module's twin
    bufs = fresh()
    eden_utils.dynamic_bitrate_bucket(x, n, *bufs[:5], bufs[5], u=u, seed=seed, step=step, strategy=strategy,
                                      stream_p=torch.cuda.current_stream().cuda_stream)
    same(bufs)
    # refusals come before any launch
    with pytest.raises(RuntimeError):
        capi.bucket_descriptor(x, n, bufs[0], bufs[1], bufs[2], bufs[3], bufs[4][:100], strategy=strategy)
    bad, dev = capi.bucket_descriptor(x, n, *bufs[:5], strategy=strategy, out=None, u=u)
    with pytest.raises(RuntimeError):
        capi.dynamic_bitrate_bucket(bad, dev)                     # the decode stage without an output
    torch.cuda.synchronize()


@pytest.mark.parametrize("streams,graphs,whole", [(1, False, False), (2, False, False), (2, True, True), (3, True, True),
                                                  (2, False, True)])
def test_single_pass_buckets_object(capi, streams, graphs, whole):
    """a stream of buckets through the pipeline object -- one host call per bucket, or a whole step recorded once and
    replayed (one graph per stream), several buckets in flight on streams of their own -- gives, on every training step,
    the outputs of the four calls with the rounding stream (seed, bucket ordinal * 2^32 + step)"""
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import SinglePassBuckets
    sizes = [256 * 123, 256 * 300, 256 * 300 - 5, 256 * 300, 256 * 77 + 1]      # (a later, larger bucket makes a stream's scratch grow)
    xs = [_llama_like(n, 40 + k) for k, n in enumerate(sizes)]
    outs = [torch.zeros_like(x) for x in xs]
    seed, u = 9, 6.0
    pipe = SinglePassBuckets(DEV, strategy=2, seed=seed, streams=streams, graphs=graphs, u=u)
    for step in range(1, 6):
        if step == 4:
            u = 7.5
            pipe.set_u(u)
        pipe.begin_step()
        for x in xs:
            x.mul_(1.25)                      # the sources change between steps; a replay must read the new values
        if whole:
            pipe.run_all(list(zip(xs, outs)))
        else:
            for x, o in zip(xs, outs):
                pipe.run(x, o)
        pipe.join()
        torch.cuda.synchronize()
        for k, (x, o) in enumerate(zip(xs, outs)):
            want = _four_calls(capi, x, x.numel(), u, 2, seed, (k << 32) + step)[5]
            assert torch.equal(bits_t(o), bits_t(want)), (step, k)


def test_streams_of_the_pipeline_object_run_side_by_side(capi):
    """dq_streams_overlap: a stream against itself never overlaps; the streams SinglePassBuckets settles on overlap
    with each other and with the caller's stream, also after the process has used up several streams of torch's pool
    (the runtime maps streams onto four hardware queues at their first use, and a queue works in order)"""
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import SinglePassBuckets
    index = torch.cuda.current_device()
    st = torch.cuda.Stream()
    assert capi.streams_overlap(st.cuda_stream, st.cuda_stream, index) is False
    with pytest.raises(RuntimeError):
        capi._check(capi.lib().dq_streams_overlap(None, None, index, None))
    scratch = torch.zeros(64, device=DEV)
    for used in range(5):
        for streams in (2, 3):
            pipe = SinglePassBuckets(DEV, strategy=2, seed=1, streams=streams, u=6.0)
            assert pipe.side_by_side and len(pipe.streams) == streams
            handles = [torch.cuda.current_stream().cuda_stream] + [s.cuda_stream for s in pipe.streams]
            assert len(set(handles)) == streams + 1
            for i in range(streams + 1):
                for j in range(i + 1, streams + 1):
                    assert capi.streams_overlap(handles[i], handles[j], index), (used, streams, i, j)
        extra = torch.cuda.Stream()              # one more stream of the pool gets its queue
        with torch.cuda.stream(extra):
            scratch.add_(1.0)
        torch.cuda.synchronize()


def test_stream_order_after_orders_two_streams(capi):
    """dq_stream_order_after: work enqueued on the waiting stream afterwards sees what the other stream had been given
    before the call -- also on the 65th and later calls, when the library's ring of events is being reused"""
    index = torch.cuda.current_device()
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    big = torch.zeros(1 << 24, device=DEV)
    flag = torch.zeros(8, device=DEV)
    seen = torch.zeros(200, 8, device=DEV)
    torch.cuda.synchronize()
    for k in range(200):
        with torch.cuda.stream(a):
            for _ in range(3):
                big.add_(1.0)                 # something for the flag's writer to queue behind
            flag.fill_(float(k + 1))
        capi.stream_order_after(b, a, index)
        with torch.cuda.stream(b):
            seen[k].copy_(flag)
        capi.stream_order_after(a, b, index)  # the next round's fill must not overtake this copy
    torch.cuda.synchronize()
    assert torch.equal(seen[:, 0].cpu(), torch.arange(1, 201, dtype=torch.float32))
    capi.stream_order_after(a, a, index)      # a stream after itself: nothing to do


@pytest.mark.parametrize("streams", [1, 2, 3])
def test_single_pass_buckets_alternating_between_recorded_and_eager_steps(capi, streams):
    """the first slot of the pipeline object runs on the caller's stream when a bucket is enqueued eagerly and on its worker
    stream when a recorded step is replayed: steps that alternate between the two (and a change of u in between) still
    give the outputs of the four calls on every step"""
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import SinglePassBuckets
    sizes = [256 * 200, 256 * 200, 256 * 120 + 3, 256 * 200, 256 * 64]
    xs = [_llama_like(n, 60 + k) for k, n in enumerate(sizes)]
    outs = [torch.zeros_like(x) for x in xs]
    seed, u = 4, 6.5
    pipe = SinglePassBuckets(DEV, strategy=2, seed=seed, streams=streams, graphs=True, u=u)
    pairs = list(zip(xs, outs))
    modes = ["all", "all", "all", "each", "all", "each", "each", "all", "each", "all"]
    x_then = [[None] * len(xs) for _ in modes]
    o_then = [[None] * len(xs) for _ in modes]
    us = []
    # no synchronisation between the steps: only the object's own ordering keeps them apart
    for step, mode in enumerate(modes, start=1):
        if step == 5:
            u = 7.25
            pipe.set_u(u)
        us.append(u)
        pipe.begin_step()
        for k, x in enumerate(xs):
            x.mul_(1.125)
            x_then[step - 1][k] = x.clone()
        if mode == "all":
            pipe.run_all(pairs)
        else:
            for x, o in pairs:
                pipe.run(x, o)
        pipe.join()
        for k, o in enumerate(outs):
            o_then[step - 1][k] = o.clone()
    torch.cuda.synchronize()
    for step, mode in enumerate(modes, start=1):
        for k in range(len(xs)):
            x = x_then[step - 1][k]
            want = _four_calls(capi, x, x.numel(), us[step - 1], 2, seed, (k << 32) + step)[5]
            assert torch.equal(bits_t(o_then[step - 1][k]), bits_t(want)), (step, mode, k)
