"""Writes tests/golden/config1_fixture.json: the fp32 oracle's loss and
per-parameter gradient norms for baseline configuration 1 (4 layers, d=256,
4 heads x 64, MLP 1024 ReLU, linear bias on, vocab 50304, ctx 256, batch 2,
tokens uniform, seed 0).  The LM head is drawn from N(0, 0.02) instead of the
reference's zeros so that gradients reach every parameter.

    python -m tests.golden.make_config1_fixture
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def build_config1():
    from oracle import ref_torch as R

    cfg = R.RefConfig(50304, 256, 256, 4, 64, 1024, 4, True, False)
    torch.manual_seed(0)
    model = R.RefTransformer(cfg)
    model.logits_out.weight.data.normal_(0.0, 0.02)
    ids = torch.randint(0, cfg.vocab_size, (2, 256))
    return cfg, model, ids


def run_config1():
    _, model, ids = build_config1()
    _, loss = model(ids, ids)
    loss.backward()
    return {
        "loss": loss.item(),
        "grad_norms": {n: p.grad.norm().item() for n, p in model.named_parameters()},
    }


if __name__ == "__main__":
    out = run_config1()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_fixture.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print(f"wrote {path}: loss {out['loss']:.6f}, {len(out['grad_norms'])} parameters")
