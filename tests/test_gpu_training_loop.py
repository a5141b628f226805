"""The optimizers inside an ordinary training loop (autograd gradients, mixed parameter groups, a learning-rate
schedule, checkpoint and resume), the way the reference's train.py uses them (train.py:424-470, 863): a small
teacher-student regression must train, and a run resumed from state_dict() must continue bit for bit."""
import copy

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


class _Net(torch.nn.Module):
    def __init__(self, d_in=128, d_h=256, d_out=64, vocab=50):
        super().__init__()
        self.emb = torch.nn.Embedding(vocab, d_in)
        self.fc1 = torch.nn.Linear(d_in, d_h, bias=True)
        self.fc2 = torch.nn.Linear(d_h, d_h, bias=False)
        self.norm = torch.nn.LayerNorm(d_h)
        self.head = torch.nn.Linear(d_h, d_out, bias=False)

    def forward(self, tok, x):
        h = self.emb(tok) + x
        h = torch.nn.functional.gelu(self.fc1(h))
        h = self.norm(h + torch.nn.functional.gelu(self.fc2(h)))
        return self.head(h)


def _groups(net, algo_kw):
    matrices = [net.fc1.weight, net.fc2.weight]
    vectors = [net.fc1.bias, net.norm.weight, net.norm.bias]
    return [dict(params=matrices, **algo_kw),
            dict(params=vectors, algorithm="adamw", lr=3e-3, weight_decay=0.0),
            dict(params=[net.emb.weight, net.head.weight], algorithm="lion", lr=3e-4)]


def _data(seed=0, n=512):
    g = torch.Generator(device=DEV).manual_seed(seed)
    tok = torch.randint(0, 50, (n,), device=DEV, generator=g)
    x = torch.randn(n, 128, device=DEV, generator=g)
    torch.manual_seed(123)
    teacher = _Net().to(DEV)
    with torch.no_grad():
        y = teacher(tok, x)
    return tok, x, y


def _train(net, opt, data, steps, sched=None):
    tok, x, y = data
    losses = []
    for _ in range(steps):
        loss = torch.nn.functional.mse_loss(net(tok, x), y)
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        if sched is not None:
            sched.step()
        losses.append(float(loss.detach()))
    return losses


@pytest.mark.parametrize("name,kw", [("Muon", dict(lr=0.02, nesterov=True)),
                                     ("Muon", dict(lr=0.02, use_polar_express=False, cautious_wd=True)),
                                     ("NorMuon", dict(lr=0.02)),
                                     ("Dion2", dict(lr=0.02, fraction=0.5)),
                                     ("NorDion2", dict(lr=0.02, fraction=0.5))])
def test_student_learns_the_teacher(name, kw):
    import dion

    torch.manual_seed(1)
    net = _Net().to(DEV)
    opt = getattr(dion, name)(_groups(net, {}), **kw)
    sched = torch.optim.lr_scheduler.LambdaLR(opt, lambda s: 1.0 - 0.5 * s / 60)
    losses = _train(net, opt, _data(), 60, sched)
    assert all(l == l and l < 1e6 for l in losses), "finite"
    assert losses[-1] < 0.5 * losses[0], (losses[0], losses[-1])
    assert sum(losses[-5:]) < sum(losses[:5])


@pytest.mark.parametrize("name,kw", [("Muon", dict(lr=0.02, nesterov=True)), ("NorMuon", dict(lr=0.02)),
                                     ("Dion2", dict(lr=0.02, fraction=0.5)),
                                     ("NorDion2", dict(lr=0.02, fraction=0.5))])
def test_resume_from_checkpoint_continues_bit_for_bit(name, kw):
    import dion

    data = _data(seed=3)
    torch.manual_seed(2)
    net_a = _Net().to(DEV)
    opt_a = getattr(dion, name)(_groups(net_a, {}), **kw)
    _train(net_a, opt_a, data, 5)
    ckpt = {"model": copy.deepcopy(net_a.state_dict()), "opt": copy.deepcopy(opt_a.state_dict())}
    _train(net_a, opt_a, data, 5)

    net_b = _Net().to(DEV)
    net_b.load_state_dict(ckpt["model"])
    opt_b = getattr(dion, name)(_groups(net_b, {}), **kw)
    opt_b.load_state_dict(ckpt["opt"])
    _train(net_b, opt_b, data, 5)
    for (ka, pa), (kb, pb) in zip(net_a.state_dict().items(), net_b.state_dict().items()):
        assert ka == kb and torch.equal(pa, pb), ka


def test_bf16_model_trains():
    """A model held in bf16 end to end (parameters, gradients, optimizer state)."""
    import dion

    torch.manual_seed(4)
    net = _Net().to(DEV).to(torch.bfloat16)
    tok, x, y = _data(seed=5)
    data = (tok, x.to(torch.bfloat16), y.to(torch.bfloat16))
    opt = dion.Muon(_groups(net, {}), lr=0.02, nesterov=True)
    losses = _train(net, opt, data, 60)
    assert all(st["momentum"].dtype == torch.bfloat16 for st in opt.state.values())
    assert losses[-1] < 0.6 * losses[0], (losses[0], losses[-1])
