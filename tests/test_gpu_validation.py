"""Every validation branch of the reference binding (eden_utils.cpp:42-53,134-146,164-172,192-209,
248-266,296-313,58-65,364-371) raises RuntimeError with the reference's text."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bufs(n=512, dt=torch.bfloat16):
    src = torch.zeros(n, dtype=dt, device=DEV)
    rnd = torch.zeros(n, dtype=dt, device=DEV)
    dst = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    return src, dst, rnd


def test_scaling_argument_errors(eden_utils):
    eu = eden_utils
    src, dst, rnd = _bufs()
    ok = (512, 4, 16, 0, 2)
    cases = [
        ((0, 4, 16, 0, 2), "n must be positive"),
        ((512, 3, 16, 0, 2), "nbits must be one of {2, 4, 8}"),
        ((512, 4, 16, 0, 4), "strategy must be 0"),
        ((512, 4, 64, 0, 2), r"chunk_size must be in \[1, 32\]"),
        ((512, 4, 12, 0, 2), "chunk_size must be a power of two"),
        ((512, 2, 2, 0, 0), "chunk_size \\* nbits must be divisible by 8"),
        ((500, 4, 16, 0, 0), "n must be a multiple of chunk_size"),
        ((16 * 17, 4, 16, 0, 2), "whole number of 16-chunk superchunks"),
    ]
    for args, msg in cases:
        with pytest.raises(RuntimeError, match=msg):
            eu.scaling_compress(src, dst, rnd, *args)
        with pytest.raises(RuntimeError, match=msg):
            eu.scaling_decompress(dst, src, *args)
        with pytest.raises(RuntimeError, match=msg):
            eu.scaling_decompress_add(dst, src, *args)
        with pytest.raises(RuntimeError, match=msg):
            eu.scaling_dec_comp(dst, src, dst.clone(), rnd, *args)
    with pytest.raises(RuntimeError, match="output must be torch.uint8"):
        eu.scaling_compress(src, src, rnd, *ok)
    with pytest.raises(RuntimeError, match="rand_pool dtype must match input dtype"):
        eu.scaling_compress(src, dst, rnd.half(), *ok)
    with pytest.raises(RuntimeError, match="input must be contiguous"):
        eu.scaling_compress(torch.zeros(1024, dtype=torch.bfloat16, device=DEV)[::2], dst, rnd, *ok)
    with pytest.raises(RuntimeError, match="input has fewer than n elements"):
        eu.scaling_compress(src[:256], dst, rnd, *ok)
    with pytest.raises(RuntimeError, match="rand_pool has fewer than n elements"):
        eu.scaling_compress(src, dst, rnd[:256], *ok)
    with pytest.raises(RuntimeError, match="output buffer is too small"):
        eu.scaling_compress(src, dst[:291], rnd, *ok)
    with pytest.raises(RuntimeError, match="input must be torch.uint8"):
        eu.scaling_decompress(src, src, *ok)
    with pytest.raises(RuntimeError, match="input buffer is too small"):
        eu.scaling_decompress(dst[:291], src, *ok)
    with pytest.raises(RuntimeError, match="output has fewer than n elements"):
        eu.scaling_decompress(dst, src[:100], *ok)
    with pytest.raises(RuntimeError, match="output must be torch.float16 or torch.bfloat16"):
        eu.scaling_decompress(dst, src.float(), *ok)
    with pytest.raises(RuntimeError, match="recv buffer is too small"):
        eu.scaling_dec_comp(dst[:291], src, dst, rnd, *ok)
    with pytest.raises(RuntimeError, match="send buffer is too small"):
        eu.scaling_dec_comp(dst, src, dst[:291], rnd, *ok)
    with pytest.raises(RuntimeError, match="inp must be torch.float16 or torch.bfloat16"):
        eu.scaling_dec_comp(dst, src.float(), dst.clone(), rnd.float(), *ok)
    with pytest.raises(RuntimeError, match="rand_pool must be a CUDA tensor"):
        eu.scaling_compress(src, dst, rnd.cpu(), *ok)
    # keyword names and defaults of the reference signature
    eu.scaling_compress(src=src, dst=dst, rand_pool=rnd, n=16 * 19, nbits=4, chunk_size=16)      # strategy=0, stream_p=0
    eu.scaling_decompress(src=dst, dst=src, n=512, nbits=4, chunk_size=16, stream_p=0, strategy=2)
    # extended entry points take what the strict ones refuse
    eu.scaling_compress_ex(src.float(), dst, rnd, 512, 5, 16, 0, 2)
    eu.scaling_decompress_ex(dst, src.float(), 512, 5, 16, 0, 2)
    torch.cuda.synchronize()


def test_superchunk_argument_errors(eden_utils):
    eu = eden_utils
    src = torch.zeros(1000, dtype=torch.bfloat16, device=DEV)
    res = torch.zeros(1024, dtype=torch.bfloat16, device=DEV)
    st = torch.zeros(8, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="stats must be torch.bfloat16"):
        eu.superchunk_mean_center(src, res, st.float(), 1000, 2)
    with pytest.raises(RuntimeError, match="residual dtype must match src dtype"):
        eu.superchunk_mean_center(src, res.half(), st, 1000, 2)
    with pytest.raises(RuntimeError, match="world_size must be positive"):
        eu.superchunk_mean_center(src, res, st, 1000, 0)
    with pytest.raises(RuntimeError, match="superchunk_size must be 256"):
        eu.superchunk_mean_center(src, res, st, 1000, 2, 128)
    with pytest.raises(RuntimeError, match="residual buffer is too small"):
        eu.superchunk_mean_center(src, res[:1000], st, 1000, 2)
    with pytest.raises(RuntimeError, match="stats buffer is too small"):
        eu.superchunk_mean_center(src, res, st[:7], 1000, 2)
    with pytest.raises(RuntimeError, match="src has fewer than n elements"):
        eu.superchunk_mean_center(src, res, st, 1001, 2)
    with pytest.raises(RuntimeError, match="src must be torch.float16 or torch.bfloat16"):
        eu.superchunk_mean_center(src.float(), res.float(), st, 1000, 2)
    with pytest.raises(RuntimeError, match="dst has fewer than n elements"):
        eu.superchunk_add_mean_copy(res, src[:10], st, 1000)
    with pytest.raises(RuntimeError, match="dst dtype must match residual dtype"):
        eu.superchunk_add_mean_copy(res, src.half(), st, 1000)
    eu.superchunk_mean_center(src=src, residual=res, stats=st, n=1000, world_size=2, superchunk_size=256, stream_p=0)
    eu.superchunk_add_mean_copy(residual=res, dst=src, stats=st, n=1000)
    torch.cuda.synchronize()


def test_packing_and_hadamard_argument_errors(eden_utils):
    eu = eden_utils
    with pytest.raises(RuntimeError, match="bins must be a torch.int32 CUDA tensor"):
        eu.EdenBinsToBits(torch.zeros(64, device=DEV), 4)
    with pytest.raises(RuntimeError, match="bins size must be a multiple of 32"):
        eu.EdenBinsToBits(torch.zeros(48, dtype=torch.int32, device=DEV), 4)
    with pytest.raises(RuntimeError, match="bins must be 1D"):
        eu.EdenBinsToBits(torch.zeros(2, 32, dtype=torch.int32, device=DEV), 4)
    with pytest.raises(RuntimeError, match="arr must be a torch.int32 CUDA tensor"):
        eu.EdenBitsToBins(torch.zeros(8, device=DEV), 4)
    with pytest.raises(RuntimeError, match="input must be 1D"):
        eu.Hadamard(torch.zeros(4, 4, device=DEV))
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        eu.Hadamard_inplace(torch.zeros(16))
    eu.Hadamard_init_ptr(0)
    eu.Hadamard_init(torch.zeros(4, dtype=torch.int32, device=DEV))
    eu.init_lookup_table()
