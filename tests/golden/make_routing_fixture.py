"""Writes routing_seed0_T8192_E32_top4.json: the per-expert routed-row counts of the benchmark
configuration (CPU generator seed 0, first draw = logits [8192, 32], top-4 of softmax)."""
import json
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from oracle import moe_ffn  # noqa: E402

logits = torch.randn(8192, 32, generator=torch.Generator().manual_seed(0))
counts, row_token, _ = moe_ffn.group_rows(moe_ffn.route_topk(logits, 4).numpy(), 32)
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "routing_seed0_T8192_E32_top4.json"), "w") as fh:
    json.dump({"tokens_per_expert": counts.tolist(), "row_token_first8_sum": int(row_token[:8].sum()),
               "made_by": "tests/golden/make_routing_fixture.py"}, fh)
