"""Writes tests/golden/sparse_modules.npz: input/output vectors of the reference's three sparse
encoder attention modules, for the parts of them that neither a third-party implementation nor a
closed form pins (T5BlockAttention as a whole; T5LocalAttention and T5TransientGlobalAttention
end to end with padded masks).

Runs only where the reference checkout is present (the build container); the reference's files
are never shipped.  It loads `src/turbot5/model/attentions.py` from the checkout on the CPU with
`use_triton=False`, so every module takes its torch ("naive") path.  Three names that the
installed `transformers` release no longer provides and that carry no arithmetic are put in
place first: the ONNX config base class that `config.py` subclasses, the `model_parallel_utils`
module (not reached from attentions.py, kept for safety) and `find_pruneable_heads_and_indices`
(head pruning, never called here).  The package's top-level `__init__` (task heads) is skipped
by registering `turbot5` as a bare namespace.

    python tests/golden/make_sparse_fixtures.py [/root/reference]

Every case stores: hidden states, attention mask, the module's weights (q, k, v, o, table and for
the transient-global module the side-token norm weight), its hyper-parameters and the module
output `forward(hidden, mask=mask)[0]` (the local module gets `_get_local_attention_mask(mask, block_len)`,
as the reference's T5Stack routes it, modeling.py:488-489).
"""
from __future__ import annotations

import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "sparse_modules.npz")


def load_reference(ref_root: str):
    src = os.path.join(ref_root, "src", "turbot5")
    if not os.path.isdir(src):
        raise SystemExit(f"no reference checkout at {ref_root}")
    import transformers
    import transformers.pytorch_utils as pu
    if not hasattr(pu, "find_pruneable_heads_and_indices"):
        def find_pruneable_heads_and_indices(*a, **k):
            raise NotImplementedError("head pruning is not part of the fixtures")
        pu.find_pruneable_heads_and_indices = find_pruneable_heads_and_indices
    if "transformers.onnx" not in sys.modules:
        try:
            import transformers.onnx  # noqa: F401
        except Exception:
            onnx = types.ModuleType("transformers.onnx")

            class OnnxSeq2SeqConfigWithPast:  # base class of T5OnnxConfig only; never instantiated
                pass
            onnx.OnnxSeq2SeqConfigWithPast = OnnxSeq2SeqConfigWithPast
            sys.modules["transformers.onnx"] = onnx
            transformers.onnx = onnx
    if "transformers.utils.model_parallel_utils" not in sys.modules:
        try:
            import transformers.utils.model_parallel_utils  # noqa: F401
        except Exception:
            mp = types.ModuleType("transformers.utils.model_parallel_utils")
            mp.assert_device_map = mp.get_device_map = lambda *a, **k: None
            sys.modules["transformers.utils.model_parallel_utils"] = mp
    for name, sub in (("turbot5", ""), ("turbot5.model", "model"), ("turbot5.ops", "ops")):
        pkg = types.ModuleType(name)
        pkg.__path__ = [os.path.join(src, sub) if sub else src]
        sys.modules[name] = pkg
    import importlib
    att = importlib.import_module("turbot5.model.attentions")
    cfg = importlib.import_module("turbot5.model.config")
    return att, cfg


def make_mask(kind: str, B: int, L: int, g: torch.Generator) -> torch.Tensor:
    m = torch.ones(B, L)
    if kind == "ones":
        return m
    if kind == "right":         # right padding, different lengths
        for b in range(B):
            n = int(torch.randint(max(1, L // 3), L, (1,), generator=g))
            m[b, n:] = 0
        return m
    if kind == "left":
        for b in range(B):
            n = int(torch.randint(1, max(2, L // 2), (1,), generator=g))
            m[b, :n] = 0
        return m
    if kind == "holes":
        m = (torch.rand(B, L, generator=g) > 0.25).float()
        m[:, 0] = 1
        return m
    raise ValueError(kind)


def run_case(att, cfgmod, cls_name, B, L, H, D, Bl, aux, mask_kind, seed):
    g = torch.Generator().manual_seed(seed)
    d_model = H * D
    config = cfgmod.T5Config(vocab_size=32, d_model=d_model, d_kv=D, d_ff=2 * d_model, num_layers=1, num_heads=H,
                             relative_attention_num_buckets=32, relative_attention_max_distance=128,
                             dropout_rate=0.0, attention_type="block", sliding_window=Bl, global_block_size=aux,
                             use_triton=False, is_decoder=False)
    mod = getattr(att, cls_name)(config, has_relative_attention_bias=True).eval()
    with torch.no_grad():
        for name, prm in mod.named_parameters():
            if name.endswith("layer_norm.weight"):
                prm.copy_(1.0 + 0.25 * torch.randn(prm.shape, generator=g))
            elif "relative_attention_bias" in name:
                prm.copy_(torch.randn(prm.shape, generator=g))
            else:   # q, k, v, o
                prm.copy_(torch.randn(prm.shape, generator=g) * (prm.shape[1] ** -0.5))
        hidden = torch.randn(B, L, d_model, generator=g)
        mask = make_mask(mask_kind, B, L, g)
        if cls_name == "T5LocalAttention":
            # the local module is handed the blocked mask that T5Stack builds (modeling.py:488-489)
            import importlib
            utils = importlib.import_module("turbot5.model.utils")
            out = mod(hidden, mask=utils._get_local_attention_mask(mask, Bl, hidden.device))[0]
        else:
            out = mod(hidden, mask=mask)[0]
    case = {"hidden": hidden, "mask": mask, "out": out,
            "meta": torch.tensor([B, L, H, D, Bl, aux], dtype=torch.int64)}
    for name, prm in mod.state_dict().items():
        case["w." + name] = prm
    return case


# (module, B, L, H, D, block_len, aux, mask)   aux = global tokens (block) / tokens per side token (transient-global)
CASES = [
    ("T5BlockAttention", 2, 64, 2, 16, 16, 4, "ones"),
    ("T5BlockAttention", 2, 40, 1, 16, 16, 8, "ones"),     # ragged last block (the reference's view() needs H == 1 for it)
    ("T5BlockAttention", 2, 10, 2, 16, 16, 4, "ones"),     # shorter than a block: full attention
    ("T5BlockAttention", 2, 48, 2, 16, 16, 16, "ones"),    # as many global tokens as a block holds
    ("T5BlockAttention", 1, 96, 3, 16, 32, 8, "ones"),
    ("T5BlockAttention", 2, 64, 2, 16, 16, 4, "right"),
    ("T5BlockAttention", 2, 40, 1, 16, 16, 8, "right"),
    ("T5LocalAttention", 2, 40, 1, 16, 16, 0, "right"),
    ("T5TransientGlobalAttention", 2, 40, 1, 16, 16, 8, "right"),
    ("T5BlockAttention", 2, 64, 2, 16, 16, 4, "left"),
    ("T5BlockAttention", 2, 64, 2, 16, 16, 4, "holes"),
    ("T5LocalAttention", 2, 64, 2, 16, 16, 0, "ones"),
    ("T5LocalAttention", 2, 64, 2, 16, 16, 0, "right"),
    ("T5LocalAttention", 2, 64, 2, 16, 16, 0, "left"),
    ("T5LocalAttention", 2, 64, 2, 16, 16, 0, "holes"),
    ("T5TransientGlobalAttention", 2, 64, 2, 16, 16, 8, "ones"),
    ("T5TransientGlobalAttention", 2, 64, 2, 16, 16, 8, "right"),
    ("T5TransientGlobalAttention", 2, 64, 2, 16, 16, 8, "left"),
    ("T5TransientGlobalAttention", 2, 64, 2, 16, 16, 8, "holes"),
    ("T5TransientGlobalAttention", 1, 96, 3, 16, 32, 16, "right"),
    # padded batches shorter than one block: full attention under a key mask (attentions.py:752, :691, :722-732)
    ("T5BlockAttention", 2, 10, 2, 16, 16, 4, "right"),
    ("T5BlockAttention", 3, 13, 2, 16, 16, 4, "holes"),
    ("T5BlockAttention", 2, 12, 2, 16, 16, 4, "left"),
]


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    att, cfgmod = load_reference(ref_root)
    blob = {}
    names = []
    for i, (cls_name, B, L, H, D, Bl, aux, mk) in enumerate(CASES):
        case = run_case(att, cfgmod, cls_name, B, L, H, D, Bl, aux, mk, seed=100 + i)
        key = f"{i:02d}.{cls_name}.{mk}"
        names.append(key)
        for k, v in case.items():
            blob[f"{key}/{k}"] = v.detach().cpu().numpy()
        print(f"{key}: B{B} L{L} H{H} D{D} Bl{Bl} aux{aux}  out {tuple(case['out'].shape)} "
              f"|out|max {case['out'].abs().max():.4f}")
    blob["cases"] = np.array(names)
    np.savez_compressed(OUT, **blob)
    print(f"wrote {OUT} ({os.path.getsize(OUT)} bytes)")


if __name__ == "__main__":
    main()
