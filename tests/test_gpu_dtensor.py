"""The DTensor worker's entry points (``get_logprobs_from_vocab_parallel_logits``,
``dtensor_from_parallel_logits_to_logprobs``) on a one-device mesh: same values as the oracle (1e-5
for fp32 logits), gradient through ``DTensor.to_local``."""

import os
import socket

import pytest
import torch

from oracle import logprob as OL

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def mesh():
    import torch.distributed as dist
    from torch.distributed.device_mesh import init_device_mesh

    own = not dist.is_initialized()
    if own:
        with socket.socket() as s:
            s.bind(("127.0.0.1", 0))
            port = s.getsockname()[1]
        os.environ["MASTER_ADDR"], os.environ["MASTER_PORT"] = "127.0.0.1", str(port)
        torch.cuda.set_device(0)
        dist.init_process_group("nccl", rank=0, world_size=1)
    try:
        yield init_device_mesh("cuda", (1, 1), mesh_dim_names=("dp", "tp"))
    finally:
        if own:
            dist.destroy_process_group()


def test_vocab_parallel_dtensor_logits(mesh):
    from torch.distributed.tensor import DTensor, Replicate, Shard

    from rl_amd.distributed import model_utils as MU

    g = torch.Generator().manual_seed(4)
    b, s, v = 3, 10, 320
    logits = torch.randn(b, s, v, generator=g) * 2
    ids = torch.randint(0, v, (b, s), generator=g)
    xo = logits.clone().requires_grad_(True)
    want = OL.next_token_logprobs(ids, xo)
    up = torch.randn(b, s - 1, generator=g)
    (want * up).sum().backward()

    x = logits.to(DEV).requires_grad_(True)
    dl = DTensor.from_local(x, mesh["tp"], [Shard(-1)])
    got = MU.get_logprobs_from_vocab_parallel_logits(dl, ids.to(DEV))
    assert got.shape == (b, s - 1)
    assert (got.detach().cpu() - want.detach()).abs().max().item() <= 1e-5
    (got * up.to(DEV)).sum().backward()
    assert (x.grad.cpu() - xo.grad).abs().max().item() <= 1e-5 * (xo.grad.abs().max().item() + 1e-30) + 1e-7

    # targets as a (replicated) DTensor, the lower-level twin, chunked
    dt = DTensor.from_local(ids.to(DEV), mesh["tp"], [Replicate()])
    with torch.no_grad():
        again = MU.dtensor_from_parallel_logits_to_logprobs(x.detach(), dt, 0, v, mesh.get_group("tp"), inference_only=True,
                                                            chunk_size=4)
    assert torch.equal(again, got.detach())
    # the front door of the loss takes the DTensor as well
    front = MU.get_next_token_logprobs_from_logits(ids.to(DEV), dl)
    assert torch.equal(front.detach(), got.detach())
    # a sequence index without a context-parallel mesh dimension trips the reference's own assertion
    with pytest.raises(AssertionError):
        MU.get_logprobs_from_vocab_parallel_logits(dl, ids.to(DEV), seq_index=torch.arange(s))
