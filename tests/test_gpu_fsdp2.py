"""GPU: the dense QLoRA modules under FSDP2 wrapping in a one-rank process group on one GPU.

Restates the world-size-1 branch of the reference's life-cycle gate
(tests/distributed/test_glm52_exact_qlora_fsdp2.py:60-141) for this package's modules: the module is a child
FSDP unit without a mixed-precision policy nested below a bf16 parent unit; after fully_shard its factors and its
packed bytes are DTensors; the packed bytes are taken out of FSDP's parameter group
(_deregister_qlora_weights_from_fsdp, qlora/utils.py:490-542) so that no policy ever casts them; the sharded
module's output bytes, dX and the full factor gradients equal the unsharded module's bit for bit.  One process,
one GPU, world size 1: no collective moves data between devices."""

import os
import socket

import pytest
import torch
import torch.distributed as dist
from torch import nn

from oracle import recipe as R
from tests.util_cases import close, gen, make_dense_module

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def one_rank_group(hip_device):
    if dist.is_initialized():
        yield
        return
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    os.environ.setdefault("HSA_ENABLE_IPC_MODE_LEGACY", "0")
    torch.cuda.set_device(0)
    dist.init_process_group(backend="nccl", init_method=f"tcp://127.0.0.1:{port}", rank=0, world_size=1,
                            device_id=hip_device)
    try:
        yield
    finally:
        dist.destroy_process_group()


class _Parent(nn.Module):
    def __init__(self, projection, device):
        super().__init__()
        self.projection = projection
        self.parent_marker = nn.Parameter(torch.ones(1, dtype=torch.float32, device=device), requires_grad=False)
        self.parent_forward_state = []

    def forward(self, x):
        from torch.distributed.tensor import DTensor

        self.parent_forward_state.append((isinstance(self.parent_marker, DTensor), self.parent_marker.dtype))
        return self.projection(x)


@pytest.mark.parametrize("fmt", ["block_fp8", "nvfp4", "int4"])
def test_fsdp2_one_rank_lifecycle(hip_device, one_rank_group, fmt):
    from torch.distributed._composable.fsdp import MixedPrecisionPolicy, fully_shard
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor import DTensor

    from xorl_amd.qlora.utils import _deregister_qlora_weights_from_fsdp

    N, K, r, M = 576 + 64, 256, 16, 17            # out_features a multiple of 64 (the backward contracts over them)
    ref_m, w_ref = make_dense_module(fmt, N, K, r, 32, seed=5, device=hip_device)
    sh_m, _ = make_dense_module(fmt, N, K, r, 32, seed=5, device=hip_device)
    reference, sharded = _Parent(ref_m, hip_device), _Parent(sh_m, hip_device)

    mesh = init_device_mesh("cuda", (1,), mesh_dim_names=("dp_shard",))
    fully_shard(sharded.projection, mesh=mesh, reshard_after_forward=True)
    fully_shard(sharded, mesh=mesh, reshard_after_forward=True,
                mp_policy=MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32))
    assert isinstance(sharded.projection.lora_A, DTensor)
    assert isinstance(sharded.projection.packed_weight_f32, DTensor)
    assert isinstance(sharded.parent_marker, DTensor)
    assert _deregister_qlora_weights_from_fsdp(sharded, param_names=("packed_weight_f32",)) == 1

    seen = []

    def record(module, _args):
        seen.append((isinstance(module.lora_A, DTensor), isinstance(module.lora_B, DTensor),
                     isinstance(module.packed_weight_f32, DTensor), module.lora_A.dtype, module.lora_B.dtype,
                     module.packed_weight_f32.dtype))

    hook = sharded.projection.register_forward_pre_hook(record)
    x = torch.linspace(-1, 1, M * K, device=hip_device, dtype=torch.bfloat16).reshape(M, K)
    dy = torch.linspace(-0.75, 0.75, M * N, device=hip_device, dtype=torch.bfloat16).reshape(M, N)
    x_ref, x_sh = x.clone().requires_grad_(True), x.clone().requires_grad_(True)

    y_ref = reference(x_ref)
    y_sh = sharded(x_sh)
    assert reference.parent_forward_state == [(False, torch.float32)]
    assert sharded.parent_forward_state == [(False, torch.bfloat16)]       # the parent's policy reaches the parent only
    # inside the forward the factors are gathered plain fp32 tensors, the packed bytes are still a (never cast) DTensor
    assert seen == [(False, False, True, torch.float32, torch.float32, torch.float32)]
    assert torch.equal(y_sh.view(torch.uint8), y_ref.view(torch.uint8))
    assert isinstance(sharded.projection.lora_A, DTensor) and isinstance(sharded.projection.packed_weight_f32, DTensor)

    y_ref.backward(dy)
    y_sh.backward(dy)
    assert torch.equal(x_sh.grad, x_ref.grad) and bool(torch.isfinite(x_sh.grad).all())
    gA, gB = sharded.projection.lora_A.grad, sharded.projection.lora_B.grad
    assert isinstance(gA, DTensor) and isinstance(gB, DTensor)
    assert torch.equal(gA.full_tensor(), reference.projection.lora_A.grad)
    assert torch.equal(gB.full_tensor(), reference.projection.lora_B.grad)
    hook.remove()

    # and the whole thing is still the right function: against the float64 program on the oracle's decode (the
    # reference test's linspace inputs give rows that cancel almost to zero: tensor-wide metric only)
    ex = R.linear_fwd_bwd_exact(x.cpu(), w_ref, ref_m.lora_A.detach().cpu(), ref_m.lora_B.detach().cpu(), ref_m.scaling, dy.cpu())
    close(y_sh.detach().cpu(), ex["y"], 1e-2, rows="none")
    close(x_sh.grad.cpu(), ex["dx"], 1e-2, rows="none")
    close(gA.full_tensor().cpu(), ex["dA"], 1e-2, rows="none")
    close(gB.full_tensor().cpu(), ex["dB"], 1e-2, rows="none")

    # decode and the byte reader gather the sharded bytes without any cast
    assert torch.equal(sharded.projection._dequantize_weight().to(torch.bfloat16).cpu(), w_ref)
    assert torch.equal(sharded.projection._read_packed_weight_uint8(), reference.projection._read_packed_weight_uint8())
