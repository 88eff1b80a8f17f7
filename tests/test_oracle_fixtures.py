"""The oracle's sparse patterns against vectors written from the reference's own modules.

`tests/golden/sparse_modules.npz` holds inputs, weights and outputs of T5BlockAttention,
T5LocalAttention and T5TransientGlobalAttention (reference src/turbot5/model/attentions.py:523-1065),
run on the CPU in the build container by `tests/golden/make_sparse_fixtures.py`.  This is the only pin of
`block_attention_blocked` against the reference module, and the pin of the local / transient-global
oracles for masks with left padding and holes.
"""
import os

import numpy as np
import pytest
import torch

from oracle import t5_basic as O

FIX = os.path.join(os.path.dirname(__file__), "golden", "sparse_modules.npz")


def load_cases():
    z = np.load(FIX, allow_pickle=False)
    out = []
    for name in z["cases"].tolist():
        c = {k.split("/", 1)[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(name + "/")}
        out.append((name, c))
    return out


CASES = load_cases()


def heads(x, H, D):
    B, L, _ = x.shape
    return x.view(B, L, H, D).transpose(1, 2)


def oracle_attention_output(name, c):
    """The module's attention op restated with the oracle's op-level functions: (B, H, L, D), head-correct, before
    the head merge and the output projection."""
    B, L, H, D, Bl, aux = (int(x) for x in c["meta"])
    hidden, mask = c["hidden"], c["mask"]
    q, k, v = (heads(hidden @ c[f"w.{n}.weight"].T, H, D) for n in ("q", "k", "v"))
    table = c["w.relative_attention_bias.weight"]
    if "Block" in name:
        return O.block_attention_blocked(q, k, v, table, Bl, aux, mask)
    if "Local" in name:
        return O.local_attention_blocked(q, k, v, table, Bl, mask)
    side = O.tglobal_side_inputs(hidden, mask, aux, c["w.global_input_layer_norm.weight"])
    sk, sv = (heads(side @ c[f"w.{n}.weight"].T, H, D) for n in ("k", "v"))
    return O.tglobal_attention_blocked(q, k, v, sk, sv, table, Bl, aux, mask)


def oracle_module_output(name, c):
    """The module's forward: the attention op above, the module's head merge and its output projection."""
    B, L, H, D, Bl, aux = (int(x) for x in c["meta"])
    o = oracle_attention_output(name, c)
    if "TransientGlobal" in name:
        # the reference module merges heads without the head transpose (attentions.py:951-953): its rows are
        # the (block, head, row-in-block) order read as (row, head).  Reproduce that here, outside the op.
        nb = -(-L // Bl) if L >= Bl else 1
        bl = Bl if L >= Bl else L
        ob = torch.zeros(B, H, nb * bl, D)
        ob[:, :, :L] = o
        ob = ob.view(B, H, nb, bl, D).permute(0, 2, 1, 3, 4).contiguous().view(B, -1, H * D)[:, :L]
        return ob @ c["w.o.weight"].T
    return o.transpose(1, 2).reshape(B, L, H * D) @ c["w.o.weight"].T


@pytest.mark.parametrize("name,c", CASES, ids=[n for n, _ in CASES])
def test_oracle_matches_reference_module(name, c):
    got = oracle_module_output(name, c)
    want = c["out"]
    # every row, padding rows included: the restatement performs the same fp32 operations in the same order
    err = (got - want).abs().max().item()
    assert err <= 1e-6, f"{name}: max-abs {err}"


def test_fixture_covers_every_module_and_mask():
    names = [n for n, _ in CASES]
    for mod in ("T5BlockAttention", "T5LocalAttention", "T5TransientGlobalAttention"):
        for mk in ("ones", "right", "left", "holes"):
            assert any(mod in n and n.endswith(mk) for n in names), (mod, mk)
