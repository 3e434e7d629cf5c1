"""``param_groups_weight_decay`` and ``to_low_precision`` (optimi/utils.py:41-71, :104-169): the
same scenarios as the reference's tests/test_weight_decay.py and tests/test_to_low_precision.py,
and, on the GPU, a mixed fp32 / bf16, decay / no-decay model stepped against the oracle."""

import warnings

import pytest
import torch
from torch import nn

import golden_util as G
import optimi_amd
from optimi_amd import param_groups_weight_decay, to_low_precision

CLASSES = [optimi_amd.Adam, optimi_amd.AdamW, optimi_amd.Lion, optimi_amd.StableAdamW, optimi_amd.Adan,
           optimi_amd.SGD, optimi_amd.RAdam, optimi_amd.Ranger]


class MLP(nn.Module):
    def __init__(self, n_in, hidden, dtype=torch.float32):
        super().__init__()
        self.fc1 = nn.Linear(n_in, hidden, bias=True, dtype=dtype)
        self.act = nn.Mish()
        self.norm = nn.LayerNorm(hidden, dtype=dtype)
        self.fc2 = nn.Linear(hidden, 1, bias=False, dtype=dtype)

    def forward(self, x):
        return self.fc2(self.norm(self.act(self.fc1(x))))


class Rope(nn.Module):
    def __init__(self):
        super().__init__()
        self.register_buffer("cos", torch.ones(4))
        self.register_buffer("sin", torch.ones(4))
        self.register_buffer("positions", torch.arange(4))  # integer: never cast


class Attention(nn.Module):
    def __init__(self, hidden):
        super().__init__()
        self.rope = Rope()
        self.q_proj = nn.Linear(hidden, hidden)
        self.v_proj = nn.Linear(hidden, hidden)

    def forward(self, x):
        return self.v_proj(self.q_proj(x))


class TinyLM(nn.Module):
    def __init__(self, vocab=128, hidden=32):
        super().__init__()
        self.tok_embeddings = nn.Embedding(vocab, hidden)
        self.attn = Attention(hidden)
        self.norm = nn.LayerNorm(hidden)
        self.head = nn.Linear(hidden, vocab)
        self.register_buffer("global_scale", torch.ones(1))

    def forward(self, x):
        return self.head(self.norm(self.attn(self.tok_embeddings(x).to(self.head.weight.dtype))))


@pytest.mark.parametrize("cls", CLASSES)
@pytest.mark.parametrize("extra", [None, "fc2"])
def test_param_groups_weight_decay(cls, extra):
    model = MLP(10, 20, torch.float16)
    groups = param_groups_weight_decay(model, weight_decay=1e-2, additional_layers=[extra] if extra else None)
    assert [g["weight_decay"] for g in groups] == [0.0, 1e-2]
    no_decay, decay = ({id(p) for p in g["params"]} for g in groups)
    want_decay = {id(model.fc1.weight)} | (set() if extra else {id(model.fc2.weight)})
    assert decay == want_decay
    assert no_decay == {id(p) for p in model.parameters()} - want_decay
    # group values win over the constructor's weight_decay
    opt = cls(groups, lr=1e-3, weight_decay=1e-3)
    assert [g["weight_decay"] for g in opt.param_groups] == [0.0, 1e-2]
    assert [len(g["params"]) for g in opt.param_groups] == [len(no_decay), len(decay)]


def test_param_groups_skip_frozen_parameters():
    model = MLP(10, 20)
    model.fc1.weight.requires_grad_(False)
    groups = param_groups_weight_decay(model)
    assert all(p is not model.fc1.weight for g in groups for p in g["params"])
    assert len(groups[1]["params"]) == 1


@pytest.mark.parametrize("cls", CLASSES)
def test_decouple_lr_warning_looks_at_groups(cls):
    model = MLP(8, 16)
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        cls([{"params": list(model.parameters()), "weight_decay": 0.0}], lr=1e-3, weight_decay=1e-2, decouple_lr=True)
    assert not caught, [str(w.message) for w in caught]
    groups = [{"params": [model.fc1.bias, model.norm.weight, model.norm.bias], "weight_decay": 0.0},
              {"params": [model.fc1.weight], "weight_decay": 2e-3}, {"params": [model.fc2.weight], "weight_decay": 5e-3}]
    with pytest.warns(UserWarning) as record:
        cls(groups, lr=1e-3, decouple_lr=True)
    assert len(record) == 1 and "0.005" in str(record[0].message) and "decouple_lr=True" in str(record[0].message)


def test_to_low_precision_defaults():
    model = to_low_precision(TinyLM(), dtype=torch.bfloat16)
    assert model.head.weight.dtype == model.attn.q_proj.bias.dtype == model.norm.weight.dtype == torch.bfloat16
    assert model.tok_embeddings.weight.dtype == torch.float32
    assert model.attn.rope.cos.dtype == model.attn.rope.sin.dtype == torch.float32
    assert model.attn.rope.positions.dtype == torch.int64
    assert model.global_scale.dtype == torch.bfloat16
    assert isinstance(model.head.weight, nn.Parameter) and model.head.weight.requires_grad


def test_to_low_precision_custom_modules():
    model = to_low_precision(TinyLM(), dtype=torch.float16, fp32_modules=(nn.LayerNorm,))
    assert model.norm.weight.dtype == model.norm.bias.dtype == torch.float32
    assert model.tok_embeddings.weight.dtype == torch.float16
    assert model.attn.rope.cos.dtype == torch.float32
    model = to_low_precision(TinyLM(), fp32_modules=None)
    assert model.tok_embeddings.weight.dtype == torch.bfloat16


def test_to_low_precision_buffer_selectors():
    model = to_low_precision(TinyLM(), fp32_buffers=())
    assert model.attn.rope.cos.dtype == torch.bfloat16 and model.tok_embeddings.weight.dtype == torch.float32
    to_low_precision(model, fp32_buffers=(Rope,))
    assert model.attn.rope.cos.dtype == model.attn.rope.sin.dtype == torch.float32
    model = to_low_precision(TinyLM(), fp32_buffers="rope")
    assert model.attn.rope.cos.dtype == torch.float32 and model.global_scale.dtype == torch.bfloat16


def test_to_low_precision_rejects_bad_selectors():
    with pytest.raises(TypeError, match="fp32_modules"):
        to_low_precision(TinyLM(), fp32_modules=("embedding",))
    with pytest.raises(TypeError, match="fp32_buffers"):
        to_low_precision(TinyLM(), fp32_buffers=(3,))


def test_to_low_precision_keeps_gradients_attached():
    model = TinyLM()
    model(torch.randint(0, 128, (2, 5))).sum().backward()
    to_low_precision(model)
    assert model.head.weight.grad is not None and model.head.weight.grad.dtype == torch.bfloat16
    assert model.tok_embeddings.weight.grad.dtype == torch.float32


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["adamw", "stableadamw", "lion"])
def test_mixed_precision_decay_groups_match_oracle(case, hip_device):
    """fp32 embeddings + bf16 everything else, split into decay / no-decay groups: every
    (group, dtype) bucket is one launch and each must match the for-loop oracle."""
    from oracle.forloop import ForLoopRun

    cls, hyper = {"adamw": (optimi_amd.AdamW, dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6)),
                  "stableadamw": (optimi_amd.StableAdamW, dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6)),
                  "lion": (optimi_amd.Lion, dict(lr=1e-4, betas=(0.9, 0.99)))}[case]
    torch.manual_seed(0)
    model = to_low_precision(TinyLM(vocab=256, hidden=64), dtype=torch.bfloat16, device=hip_device)
    groups = param_groups_weight_decay(model, weight_decay=1e-2)
    assert {p.dtype for g in groups for p in g["params"]} == {torch.float32, torch.bfloat16}
    opt = cls(groups, **hyper)
    refs = []
    for g in groups:  # the oracle holds one dtype-uniform list per run
        for dt in (torch.float32, torch.bfloat16):
            ps = [p for p in g["params"] if p.dtype == dt]
            if ps:
                refs.append((ps, ForLoopRun(case, [p.detach().cpu().clone() for p in ps], weight_decay=g["weight_decay"], **hyper)))
    gen = torch.Generator().manual_seed(1)
    for _ in range(10):
        x = torch.randint(0, 256, (8, 16), generator=gen).to(hip_device)
        model(x).float().pow(2).mean().backward()
        for ps, ref in refs:
            ref.step([p.grad.detach().cpu().clone() for p in ps])
        opt.step()
        opt.zero_grad()
    for ps, ref in refs:
        for i, p in enumerate(ps):
            G.assert_close_to_reference(p.detach().flatten(), ref.params[i].flatten(), f"{case} param {tuple(p.shape)} {p.dtype}", is_param=True)
            G.assert_close_to_reference(opt.state[p]["exp_avg"].flatten(), ref.state[i]["exp_avg"].flatten(), f"{case} exp_avg {tuple(p.shape)}")
