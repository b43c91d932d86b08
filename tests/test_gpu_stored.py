"""A pre-quantized checkpoint (`quant.stored`) loaded onto the GPU: the attached bases bind to the
HIP `fp8_linear`, keep no 16-bit weight, and give the output of a base quantized on the GPU
from the dense weight (the GPU quantizers equal the host's byte for byte)."""

import pytest
import torch
from torch import nn

from kohakumosstrainer_amd.kernels import registry
from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant import stored
from kohakumosstrainer_amd.quant.compute import ComputeWeight
from oracle import formats, linear
from oracle.stats import rel_l2

pytestmark = pytest.mark.gpu


class Two(nn.Module):
    def __init__(self):
        super().__init__()
        self.up = MossLinear(256, 512, bias=True)
        self.down = MossLinear(512, 256, bias=False)
        for lin in (self.up, self.down):
            lin.init_weights(0.05)
        nn.init.normal_(self.up.bias, std=0.1)

    def forward(self, x):
        return self.down(torch.nn.functional.gelu(self.up(x)))


@pytest.mark.parametrize("recipe", ("mx", "row", "block", "tensor"))
def test_stored_checkpoint_runs_on_the_hip_backend(tmp_path, recipe):
    registry.load_backends()
    torch.manual_seed(0)
    src = Two()
    dense_up = src.up.weight.detach().clone()
    for lin in (src.up, src.down):
        lin.set_base(ComputeWeight.from_weight(lin.weight.detach().to(torch.bfloat16), recipe))
    path = tmp_path / "two.safetensors"
    stored.save_quantized(src, path, torch.bfloat16)

    model = Two()
    assert stored.load_quantized(model, path, "cuda", torch.bfloat16) == 2
    assert model.up.weight.numel() == 0 and model.up.base.q.is_cuda and model.up.base.q.dtype == torch.float8_e4m3fn
    on_gpu = ComputeWeight.from_weight(dense_up.to(torch.bfloat16).cuda(), recipe)
    assert torch.equal(on_gpu.q.view(torch.uint8), model.up.base.q.view(torch.uint8)), "GPU quantizer == stored host codes"
    assert torch.equal(on_gpu.scale.cpu(), model.up.base.scale.cpu())

    x = torch.randn(300, 256).to(torch.bfloat16)
    y = model.up(x.cuda())
    xq, xs = formats.quantize(x, recipe, "act")
    truth = linear.exact64(xq, xs, recipe) @ linear.exact64(src.up.base.q, src.up.base.scale, recipe).T + src.up.bias.double()
    assert y.dtype == torch.bfloat16 and rel_l2(y.cpu(), truth) <= 2e-3
    assert torch.isfinite(model(x.cuda())).all()


@pytest.mark.parametrize("recipe,dgrad", (("mx", True), ("mx", False), ("row", False)))
def test_streamed_slot_view_on_the_hip_backend(recipe, dgrad):
    """A streamed fp8 base on the card: the slot is refilled with another layer between forward and
    backward; output and gradients equal the resident base's bit for bit (with `dgrad` off the input
    gradient is the 16-bit kernel over the slot's codes)."""
    from kohakumosstrainer_amd.quant.compute import StreamedParts

    registry.load_backends()
    g = torch.Generator().manual_seed(1)
    make = lambda: ComputeWeight.from_weight((torch.randn(384, 256, generator=g) * 0.05).to(torch.bfloat16).cuda(), recipe, dgrad)
    layer_a, layer_b = make(), make()
    slot = {name: t.clone() for name, t in layer_a.tensors().items()}

    def fetch_a():
        for name, t in layer_a.tensors().items():
            slot[name].copy_(t)
        return slot

    view = StreamedParts(recipe, fetch_a, torch.bfloat16, "cuda")
    x = torch.randn(200, 256, generator=g).to(torch.bfloat16).cuda().requires_grad_()
    bias = torch.randn(384, generator=g).to(torch.bfloat16).cuda().requires_grad_()
    dy = torch.randn(200, 384, generator=g).to(torch.bfloat16).cuda()
    y = view.linear(x, bias)
    for name, t in layer_b.tensors().items():
        slot[name].copy_(t)
    y.backward(dy)
    x2, b2 = x.detach().clone().requires_grad_(), bias.detach().clone().requires_grad_()
    y2 = layer_a.linear(x2, b2)
    y2.backward(dy)
    assert torch.equal(y.detach(), y2.detach())
    assert torch.equal(x.grad, x2.grad) and torch.equal(bias.grad, b2.grad)
