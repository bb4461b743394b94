"""Seeded random differential test: a few hundred random shapes (element type, chunk size, code width, strategy, length,
pointer misalignment, value range, special values) through compress / decompress / decompress_add / dec_comp, every byte
against the oracle.  The cases are fixed by the seed, so a failure names a reproducible case."""
import numpy as np
import pytest
import torch

from helpers import BF16, F16, F32, TORCH_DT, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        dt = int(rng.choice([F16, BF16, F32]))
        C = int(rng.choice([16, 16, 16, 16, 8, 32, 4, 2, 1]))
        nbits = int(rng.choice([2, 3, 4, 5, 6, 7, 8]))
        strategy = int(rng.integers(0, 4))
        if (C * nbits) % 8:
            continue
        if strategy >= 2:
            n = C * 16 * int(rng.integers(1, 70))
        else:
            n = C * int(rng.integers(1, 900))
        out.append(dict(dt=dt, C=C, nbits=nbits, strategy=strategy, n=n, src_off=int(rng.integers(0, 9)),
                        rnd_off=int(rng.integers(0, 9)), enc_off=int(rng.integers(0, 17)), out_off=int(rng.integers(0, 9)),
                        scale_exp=int(rng.integers(-30, 8)) if dt != F16 else int(rng.integers(-12, 6)),
                        special=bool(rng.random() < 0.3), seed=int(rng.integers(0, 1 << 30))))
    return out


CASES = _cases(20260101, 240)


def _same(got, want):
    got, want = np.asarray(got), np.asarray(want)
    if got.dtype == np.float32:
        nan = np.isnan(got) & np.isnan(want)
        return ((got.view(np.uint32) == want.view(np.uint32)) | nan).all()
    return (got == want).all()


@pytest.mark.parametrize("k", range(0, len(CASES), 8))
def test_random_shapes(capi, oracle, k):
    for case in CASES[k:k + 8]:
        dt, C, nbits, strategy, n = case["dt"], case["C"], case["nbits"], case["strategy"], case["n"]
        tdt = TORCH_DT[dt]
        g = torch.Generator().manual_seed(case["seed"])
        src = torch.randn(n, generator=g) * (2.0 ** case["scale_exp"])
        if case["special"]:
            idx = torch.randint(0, n, (max(1, n // 50),), generator=g)
            vals = torch.tensor([0.0, float("inf"), float("-inf"), float("nan"), 1e30, -1e-30, 65504.0])
            src[idx] = vals[torch.randint(0, vals.numel(), idx.shape, generator=g)]
        src = src.to(tdt)
        rnd = torch.rand(n, generator=g)
        rnd[::5] = 0.0
        rnd[2::9] = 1.0
        rnd = rnd.to(tdt)
        base = (torch.randn(n, generator=g) * (2.0 ** case["scale_exp"])).to(tdt)
        nbytes = oracle.required_bytes(n, nbits, C, strategy)

        def view(t, off, fill=0):
            buf = torch.full((t.numel() + 24,), fill, dtype=t.dtype, device=DEV)
            v = buf[off:off + t.numel()]
            v.copy_(t)
            return buf, v

        _, src_d = view(src, case["src_off"])
        _, rnd_d = view(rnd, case["rnd_off"])
        enc_buf = torch.full((nbytes + 40,), 0x5A, dtype=torch.uint8, device=DEV)
        enc_d = enc_buf[case["enc_off"]:case["enc_off"] + nbytes]
        tag = str(case)
        capi.scaling_compress(src_d, enc_d, rnd_d, n, nbits, C, strategy)
        enc_o = oracle.scaling_compress(to_bits(src), to_bits(rnd), n, nbits, C, strategy, dt)
        got = enc_buf.cpu().numpy()
        assert (got[case["enc_off"]:case["enc_off"] + nbytes] == enc_o).all(), tag
        assert (got[:case["enc_off"]] == 0x5A).all() and (got[case["enc_off"] + nbytes:] == 0x5A).all(), tag

        out_buf, out_d = view(torch.zeros(n, dtype=tdt), case["out_off"], fill=3)
        capi.scaling_decompress(enc_d, out_d, n, nbits, C, strategy)
        dec_o = np.zeros(n, np.float32 if dt == F32 else np.uint16)
        oracle.scaling_decompress(enc_o, dec_o, n, nbits, C, strategy, dt)
        assert _same(to_bits(out_d), dec_o), tag
        ob = out_buf.float().cpu()
        assert (ob[:case["out_off"]] == 3).all() and (ob[case["out_off"] + n:] == 3).all(), tag

        _, add_d = view(base, case["out_off"])
        capi.scaling_decompress(enc_d, add_d, n, nbits, C, strategy, add=True)
        add_o = to_bits(base)
        oracle.scaling_decompress(enc_o, add_o, n, nbits, C, strategy, dt, add=True)
        assert _same(to_bits(add_d), add_o), tag

        _, inp_d = view(base, case["src_off"])
        send_d = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        capi.scaling_dec_comp(enc_d, inp_d, send_d, rnd_d, n, nbits, C, strategy)
        inp_o = to_bits(base)
        send_o = oracle.scaling_dec_comp(enc_o, inp_o, to_bits(rnd), n, nbits, C, strategy, dt)
        assert (send_d.cpu().numpy() == send_o).all(), tag
        assert _same(to_bits(inp_d), inp_o), tag
