"""Writes tests/golden/c3_lengths.json: the 32 sequence lengths of the packed variable-length workload
(uniform in [128, 4096], seed 1), so that its definition cannot drift between torch versions."""
import json
import os

import torch

lens = torch.randint(128, 4097, (32,), generator=torch.Generator().manual_seed(1)).tolist()
out = {"definition": "torch.randint(128, 4097, (32,), generator=torch.Generator().manual_seed(1))", "lengths": lens,
       "total": sum(lens)}
json.dump(out, open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "c3_lengths.json"), "w"), indent=1)
