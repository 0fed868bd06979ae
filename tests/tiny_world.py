"""Loader of the hand-derived two-rank world in tests/golden/ll_tiny_world.json (CPU and GPU suites)."""
import json
import os

import torch


def load_tiny_world():
    with open(os.path.join(os.path.dirname(__file__), "golden", "ll_tiny_world.json")) as f:
        g = json.load(f)
    h = g["hidden"]
    x_all = [torch.tensor(v, dtype=torch.float32).view(-1, 1).expand(-1, h).to(torch.bfloat16).contiguous()
             for v in g["x_value"]]
    topk_all = [torch.tensor(v, dtype=torch.int64) for v in g["topk_idx"]]
    return g, x_all, topk_all


def tiny_world_expected(g, key):
    want = g["dispatch"][key]
    begin, cnt = torch.tensor(want["layout_range_begin"]), torch.tensor(want["layout_range_count"])
    layout = torch.where(cnt > 0, (begin << 32) | cnt, torch.zeros_like(cnt))
    return want, layout
