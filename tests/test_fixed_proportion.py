"""Fixed-proportion bit-width allocation (comm_hooks.py:710-721, :842-856), CPU side: the oracle's stable
descending argsort against torch's own on the CPU, and the host mirror against the oracle."""
import numpy as np
import pytest
import torch

from helpers import to_bits


def _bf16_bits(t):
    return to_bits(t.to(torch.bfloat16))


def _norm_sets():
    g = torch.Generator().manual_seed(11)
    sets = {}
    sets["lognormal"] = torch.exp(torch.randn(5000, generator=g) * 3 - 8).to(torch.bfloat16)
    sets["few values"] = torch.tensor([1.0, 0.5, 0.25, 2.0])[torch.randint(0, 4, (3001,), generator=g)].to(torch.bfloat16)
    sets["one value"] = torch.full((257,), 3.0).to(torch.bfloat16)
    sets["single"] = torch.tensor([7.0]).to(torch.bfloat16)
    sp = torch.exp(torch.randn(2000, generator=g) * 4 - 5).to(torch.bfloat16)
    sp[::7] = 0.0
    sp[3::11] = -0.0
    sp[1::97] = float("nan")
    sp[2::131] = -1.0
    sp[5::173] = float("inf")
    sp[6::191] = float("-inf")
    sets["zeros, NaN, infinities, negatives"] = sp
    neg_nan = sp.clone().view(torch.int16)
    neg_nan[1::97] = torch.tensor(0xFFC1 - 0x10000, dtype=torch.int16)      # NaN with the sign bit set
    sets["NaN of either sign"] = neg_nan.view(torch.bfloat16)
    return sets


@pytest.mark.parametrize("name", sorted(_norm_sets()))
def test_oracle_argsort_matches_torch_cpu(oracle, name):
    norms = _norm_sets()[name]
    want = torch.argsort(norms.float(), descending=True, stable=True).numpy()
    got = oracle.argsort_descending_stable(_bf16_bits(norms))
    assert (got == want).all()
    # interleaved statistics: the norm is the second of every pair
    st = torch.zeros((norms.numel(), 2), dtype=torch.bfloat16)
    st[:, 0] = 0.25
    st[:, 1] = norms
    assert (oracle.argsort_descending_stable(_bf16_bits(st.reshape(-1))[1:], stride=2) == want).all()


def test_oracle_argsort_properties(oracle):
    bits = np.array([0x3f80, 0x7fc0, 0x0000, 0x8000, 0x3f80, 0xbf80, 0x7f80, 0xff80, 0x0000], np.uint16)
    #               1.0     NaN     +0      -0      1.0     -1.0    +inf    -inf    +0
    assert oracle.argsort_descending_stable(bits).tolist() == [1, 6, 0, 4, 2, 3, 8, 5, 7]
    assert oracle.argsort_descending_stable(np.zeros(0, np.uint16)).size == 0


def test_thresholds_and_counts():
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    T = B.fixed_proportion_thresholds
    assert T("dynamiQ_mee_5bit") == {8: 0.35, 4: 0.45, 2: 0.2}
    assert T("dynamiQ_aee") == {8: 0.35, 4: 0.45, 2: 0.2}
    assert T("dynamiQ_mee_4bit") == {8: 0.05, 4: 0.6, 2: 0.35}
    assert T("dynamiQ_mee_4bit_fixed") == {4: 1, 8: 0, 2: 0}
    assert T("dynamiQ_mee_3bit") == {8: 1 / 40, 4: 13 / 40, 2: 26 / 40}
    assert T("dynamiQ_mee_6bit") == {8: 0.55, 4: 0.35, 2: 0.1}
    assert T("dynamiQ_mee_7bit") == {8: 0.75, 4: 0.22, 2: 0.03}
    assert T("dynamiQ_3bit_4bit") == T("x_4bit")                       # "4bit" is tested first (comm_hooks.py:844)
    C = B.fixed_proportion_counts
    assert C(25600, T("x_5bit")) == (8960, 11520, 5120)
    assert C(25600, T("x_3bit")) == (640, 8320, 16640)
    assert C(25600, T("x_4bit_fixed")) == (0, 25600, 0)
    assert C(7, T("x_5bit")) == (2, 4, 1)                              # int() truncates 2.45 and 1.4
    assert C(1, T("x_7bit")) == (0, 1, 0)
    assert C(10, {8: 0.7, 4: 0.0, 2: 0.6}) == (7, 0, 3)                # the 2-bit share gives way
    for nsc in (1, 2, 3, 99, 100, 25600, 65535):
        for m in ("a", "a_3bit", "a_4bit", "a_4bit_fixed", "a_6bit", "a_7bit"):
            top, mid, bottom = C(nsc, T(m))
            assert top >= 0 and mid >= 0 and bottom >= 0 and top + mid + bottom == nsc


@pytest.mark.parametrize("method", ["a_5bit", "a_3bit", "a_4bit", "a_4bit_fixed", "a_6bit", "a_7bit"])
def test_host_groups_match_oracle(oracle, method):
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    thr = B.fixed_proportion_thresholds(method)
    for name, norms in sorted(_norm_sets().items()):
        top, mid, bottom = B.fixed_proportion_counts(norms.numel(), thr)
        g8, g4, g2 = B.fixed_proportion_groups(norms, thr)
        o8, o4, o2 = oracle.fixed_proportion_groups(_bf16_bits(norms), top, bottom)
        assert (g8.numpy() == o8).all() and (g4.numpy() == o4).all() and (g2.numpy() == o2).all(), name
        assert (g8.numel(), g4.numel(), g2.numel()) == (top, mid, bottom)


def test_capi_refuses_host_tensors():
    """a CPU tensor, a strided view or a non-tensor must raise before the library is entered: the kernels would
    dereference a host address"""
    from dynamiq_sigcomm_artifact_amd import capi
    capi.lib()
    x = torch.zeros(256, dtype=torch.bfloat16)
    dst = torch.zeros(146, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        capi.scaling_compress(x, dst, x, 256, 4, 16, 2, stream=0)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        capi.rht_blocked(torch.zeros(64), None, 64, 1.0, stream=0)
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        capi.eden_dequantize(torch.zeros(8, dtype=torch.int32), 64, torch.zeros(16), 4, torch.zeros(64), stream=0)
    with pytest.raises(RuntimeError, match="tensor argument is required"):
        capi.scaling_decompress(dst.numpy(), x, 256, 4, 16, 2, stream=0)
