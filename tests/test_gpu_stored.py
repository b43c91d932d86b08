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
