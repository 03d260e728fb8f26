"""The counter-based input generator: known answers of the hash, moments of the normal draw, and
(on a GPU) bit-equality between CPU and GPU."""
import pytest
import torch

from rl_kernel_amd import synthetic as S


def test_splitmix64_known_answers():
    # the published test vector of splitmix64 seeded with 0: first outputs of the sequence
    # state += golden; mix(state)  ==  splitmix64(0), splitmix64(golden), ...
    golden = -7046029254386353131
    wrap = lambda v: (v + (1 << 63)) % (1 << 64) - (1 << 63)
    got = [int(S.splitmix64(torch.tensor([wrap(k * golden)], dtype=torch.int64))[0]) & 0xFFFFFFFFFFFFFFFF
           for k in range(3)]
    assert got == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]


def test_values_are_a_function_of_seed_tensor_and_index():
    a = S.normal(1002, 0, (1000, 64))
    b = S.normal(1002, 0, (64000,))
    assert torch.equal(a.reshape(-1), b)                                  # shape does not matter
    assert torch.equal(S.normal(1002, 0, (70000,), chunk=4096)[:64000], b)  # nor does chunking
    assert not torch.equal(S.normal(1002, 1, (64000,)), b) and not torch.equal(S.normal(1003, 0, (64000,)), b)
    x = S.normal(7, 3, (1 << 20,))
    assert abs(x.mean().item()) < 4e-3 and abs(x.var().item() - 1.0) < 1e-2 and x.abs().max().item() <= 6.0
    assert abs((x.abs() < 1.0).float().mean().item() - 0.6827) < 5e-3
    w = S.normal(7, 4, (1 << 18,), std=0.02, dtype=torch.bfloat16)
    assert w.dtype == torch.bfloat16 and abs(w.float().std().item() - 0.02) < 5e-4
    t = S.randint(7, 5, (100000,), 128256)
    assert t.dtype == torch.int64 and int(t.min()) >= 0 and int(t.max()) < 128256 and t.unique().numel() > 60000
    m = S.bernoulli(7, 6, (1 << 20,), 0.01)
    assert abs(m.float().mean().item() - 0.01) < 1e-3


@pytest.mark.gpu
def test_cpu_and_gpu_draw_the_same_bits():
    dev = torch.device("cuda:0")
    for dtype, std in ((torch.float32, 1.0), (torch.bfloat16, 0.02), (torch.float16, 1.0)):
        assert torch.equal(S.normal(11, 2, (513, 257), std=std, dtype=dtype),
                           S.normal(11, 2, (513, 257), std=std, dtype=dtype, device=dev).cpu())
    assert torch.equal(S.randint(11, 3, (100000,), 151936), S.randint(11, 3, (100000,), 151936, device=dev).cpu())
    assert torch.equal(S.bernoulli(11, 4, (100000,), 0.01), S.bernoulli(11, 4, (100000,), 0.01, device=dev).cpu())
