"""The Mamba-2 and Mamba-1 stacks of ssm_amd.harness on the GPU: cached single-token decoding must reproduce
the logits of one forward over the whole sequence (conv window and SSM state hand-off), eagerly
and through a captured graph."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def small(kind="mamba2"):
    from ssm_amd.harness import Mamba1Config, Mamba1LM, Mamba2Config, Mamba2LM
    if kind == "mamba1":
        return Mamba1LM(Mamba1Config(d_model=128, n_layer=2, expand=2, d_state=16, d_conv=4, vocab_size=512), seed=3)
    cfg = Mamba2Config(d_model=128, n_layer=2, expand=2, headdim=64, d_state=64, ngroups=1, d_conv=4,
                       chunk_size=64, vocab_size=512)
    return Mamba2LM(cfg, seed=3)


@pytest.mark.parametrize("kind", ["mamba2", "mamba1"])
def test_prefill_then_steps_reproduce_the_full_forward(kind):
    model = small(kind)
    g = torch.Generator().manual_seed(1)
    tokens = torch.randint(0, 512, (2, 136), generator=g).cuda()
    with torch.no_grad():
        full = model.forward(tokens).float()                             # ragged length: five-kernel SSD path
        logits, cache = model.forward(tokens[:, :128], return_cache=True)   # one-pass SSD path
        torch.testing.assert_close(logits.float(), full[:, :128], rtol=3e-2, atol=3e-2 * float(full.abs().max()))
        for t in range(128, 136):
            step = model.step(tokens[:, t], cache).float()
            torch.testing.assert_close(step, full[:, t], rtol=3e-2, atol=3e-2 * float(full.abs().max()),
                                       msg=lambda m: f"position {t}: {m}")


@pytest.mark.parametrize("kind", ["mamba2", "mamba1"])
def test_short_prompt_pads_the_conv_window(kind):
    model = small(kind)
    tokens = torch.tensor([[5, 9]]).cuda()
    with torch.no_grad():
        full = model.forward(torch.tensor([[5, 9, 11]]).cuda()).float()
        _, cache = model.forward(tokens, return_cache=True)
        step = model.step(torch.tensor([11]).cuda(), cache).float()
    torch.testing.assert_close(step, full[:, 2], rtol=3e-2, atol=3e-2 * float(full.abs().max()))


@pytest.mark.parametrize("kind", ["mamba2", "mamba1"])
def test_graph_replay_generates_what_eager_stepping_generates(kind):
    model = small(kind)
    g = torch.Generator().manual_seed(2)
    tokens = torch.randint(0, 512, (2, 64), generator=g).cuda()
    eager, _ = model.generate(tokens, 12, use_graph=False)
    graphed, _ = model.generate(tokens, 12, use_graph=True)
    assert torch.equal(eager, graphed)
