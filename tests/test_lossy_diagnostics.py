"""Host-side lossy diagnostics (subspec_amd.lossy_diagnostics) against the reference-written
golden vectors: fed with per-node arrays computed by plain torch, they must reproduce every
exported metric.  No GPU."""
import json
import math
import os

import pytest
import torch

from subspec_amd.cpu_tree import Tree
from subspec_amd.lossy_diagnostics import record_lossy_diagnostics
from subspec_amd.wandb_logger import wandb_logger

GOLD = os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


class _ArrayTree:
    def __init__(self, tokens, parents):
        self.t, self.p = tokens, parents

    def get_tree_data(self, skip_nodes=0):
        return {"token_ids": torch.tensor(self.t[skip_nodes:]), "parent_indices": torch.tensor(self.p[skip_nodes:])}


@pytest.mark.parametrize("idx", range(40))
def test_diagnostics_match_reference(idx):
    with open(GOLD) as f:
        c = json.load(f)["lossy"][idx]
    probs = torch.softmax(torch.tensor(c["logits"]).to(DT[c["dtype"]]), -1)
    V = probs.shape[1]
    target = probs.argmax(-1)
    entropy = (torch.special.entr(probs).sum(-1) / math.log(V)).float()
    child_prob = torch.tensor([float(probs[p, t]) if p >= 0 else -1.0 for p, t in zip(c["parents"], c["token_ids"])])
    wandb_logger.clear_log_data()
    record_lossy_diagnostics(
        tree=_ArrayTree(c["token_ids"], c["parents"]), skip_nodes=0, target=target, entropy=entropy,
        child_prob=child_prob, tokens=torch.tensor(c["sampled"]), contexts=torch.tensor(c["hidden"]),
        accept_len=c["accept_len"], eos_token_id=c["eos_token_id"], threshold=c["threshold"],
        window_size=c["window_size"], threshold_method=c["threshold_method"])
    for key, val in c["log"].items():
        got = wandb_logger.log_data[key]
        if isinstance(val, str):
            assert got == val
        else:
            assert abs(got - val) < 1e-6, (key, got, val)
