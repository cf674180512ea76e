"""sdv2_rms_norm (WanRMSNorm.forward, wan_base/modules/model.py:77-86) against
the torch expression evaluated on the CPU, which the oracle's wan_rms_norm
restates: bit for bit, for the widths of the models and awkward ones."""
import pytest
import torch

from oracle import sdv2_oracle as oracle
from streamdiffusionv2_amd import ops
from streamdiffusionv2_amd.attention import WanRMSNorm


def _bits(t):
    return t.contiguous().view(torch.int16 if t.dtype == torch.bfloat16 else torch.int32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("width,tokens", [(1536, 1560), (5120, 777), (256, 24), (640, 33), (8192, 9), (6144, 5),
                                          (128, 3)])
def test_bit_exact_against_the_torch_expression_on_the_cpu(gpu_device, dtype, width, tokens):
    print(f"rms norm width={width} tokens={tokens} {dtype}", flush=True)
    gen = torch.Generator().manual_seed(width + tokens)
    x = (torch.randn(2, tokens, width, generator=gen) * 3.0).to(dtype)
    weight = (torch.rand(width, generator=gen) + 0.5).to(dtype)
    want = oracle.wan_rms_norm(x, weight, 1e-6)
    got = ops.rms_norm(x.to(gpu_device), weight.to(gpu_device), 1e-6)
    assert got.shape == x.shape and got.dtype == dtype and got.is_contiguous()
    assert torch.equal(_bits(got.cpu()), _bits(want))


@pytest.mark.gpu
def test_rows_inside_a_wider_tensor_and_in_place(gpu_device):
    """The q third of a packed q / k / v projection output is normalised where
    it lies; the two other thirds and whatever lies between the rows of the
    output stay untouched."""
    print("rms norm on a slice, in place", flush=True)
    gen = torch.Generator().manual_seed(11)
    width, tokens = 1536, 100
    packed = (torch.randn(1, tokens, 3 * width, generator=gen) * 2.0).bfloat16()
    weight = (torch.rand(width, generator=gen) + 0.5).bfloat16()
    want = oracle.wan_rms_norm(packed[..., width:2 * width], weight, 1e-6)
    dev = packed.to(gpu_device)
    got = ops.rms_norm(dev[..., width:2 * width], weight.to(gpu_device), 1e-6)
    assert got.is_contiguous() and torch.equal(_bits(got.cpu()), _bits(want))
    assert torch.equal(_bits(dev.cpu()), _bits(packed))                       # the input is only read
    out = ops.rms_norm(dev[..., width:2 * width], weight.to(gpu_device), 1e-6, out=dev[..., width:2 * width])
    assert out.data_ptr() == dev[..., width:2 * width].data_ptr()
    after = dev.cpu()
    assert torch.equal(_bits(after[..., width:2 * width]), _bits(want))
    assert torch.equal(_bits(after[..., :width]), _bits(packed[..., :width]))
    assert torch.equal(_bits(after[..., 2 * width:]), _bits(packed[..., 2 * width:]))


@pytest.mark.gpu
def test_fp32_rows_inside_a_wider_tensor(gpu_device):
    print("rms norm on an fp32 slice", flush=True)
    gen = torch.Generator().manual_seed(13)
    width, tokens = 640, 37
    wide = torch.randn(3, tokens, 2 * width, generator=gen) * 4.0
    weight = torch.rand(width, generator=gen) + 0.5
    want = oracle.wan_rms_norm(wide[..., width:], weight, 1e-5)
    dev = wide.to(gpu_device)
    got = ops.rms_norm(dev[..., width:], weight.to(gpu_device), 1e-5)
    assert torch.equal(_bits(got.cpu()), _bits(want))
    ops.rms_norm(dev[..., width:], weight.to(gpu_device), 1e-5, out=dev[..., :width])      # into the other half
    after = dev.cpu()
    assert torch.equal(_bits(after[..., :width]), _bits(want))
    assert torch.equal(_bits(after[..., width:]), _bits(wide[..., width:]))


@pytest.mark.gpu
def test_the_module_uses_the_kernel_and_keeps_the_expression_elsewhere(gpu_device):
    print("WanRMSNorm module", flush=True)
    torch.manual_seed(12)
    norm = WanRMSNorm(1536, eps=1e-6).to(gpu_device).bfloat16()
    with torch.no_grad():
        norm.weight.uniform_(0.5, 1.5)
    x = (torch.randn(1, 50, 1536, device=gpu_device) * 2.0).bfloat16()
    want = oracle.wan_rms_norm(x.cpu(), norm.weight.detach().cpu(), 1e-6)
    with torch.inference_mode():
        got = norm(x)
    assert torch.equal(_bits(got.cpu()), _bits(want))
    # autograd on: the torch expression, with its graph
    y = norm(x)
    assert y.requires_grad and (y.float().cpu() - want.float()).abs().max().item() <= 2e-2
    # a width the kernel does not take: the expression
    odd = WanRMSNorm(200).to(gpu_device).bfloat16()
    with torch.inference_mode():
        z = odd(torch.randn(3, 200, device=gpu_device).bfloat16())
    assert z.shape == (3, 200)


@pytest.mark.gpu
def test_argument_errors(gpu_device):
    print("rms norm argument errors", flush=True)
    x = torch.zeros(4, 256, device=gpu_device, dtype=torch.bfloat16)
    w = torch.ones(256, device=gpu_device, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.rms_norm(x, w.float(), 1e-6)                              # weight of another dtype
    with pytest.raises(RuntimeError):
        ops.rms_norm(torch.zeros(4, 200, device=gpu_device, dtype=torch.bfloat16), w[:200], 1e-6)
    with pytest.raises(RuntimeError):
        ops.rms_norm(x.cpu(), w.cpu(), 1e-6)                          # no CPU path
    with pytest.raises(RuntimeError):
        ops.rms_norm(x.t().contiguous().t(), w, 1e-6)                  # rows not contiguous
    with pytest.raises(RuntimeError):
        ops.rms_norm(x, w, 1e-6, out=torch.zeros(4, 256, device=gpu_device))      # out of another dtype
    assert ops.rms_norm(x[:0], w, 1e-6).shape == (0, 256)             # nothing to do
