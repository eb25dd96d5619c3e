"""Loads the golden fixtures of tests/golden (inputs and expected outputs frozen from the CPU oracle)."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _t16(a, dtype):
    return torch.from_numpy(a.view(np.int16).copy()).view(dtype)


def load_sfa_small():
    z = np.load(os.path.join(GOLDEN, "sfa_small.npz"))
    case = {
        "b": 2, "s1": 2, "nq": 16, "topk": 128, "block_size": 128, "softmax_scale": float(z["softmax_scale"]),
        "act_seq": z["act_seq"].tolist(), "q": _t16(z["q"], torch.bfloat16), "kn": torch.from_numpy(z["kn"].copy()),
        "kr": _t16(z["kr"], torch.bfloat16), "kn_scales": torch.from_numpy(z["kn_scales"].copy()),
        "topk_indices": torch.from_numpy(z["topk_indices"].copy()),
        "block_table": torch.from_numpy(z["block_table"].copy()),
    }
    expect = {"no_flash": _t16(z["out_no_flash"], torch.bfloat16), "flash64": _t16(z["out_flash64"], torch.bfloat16)}
    return case, expect


def load_indexer_small():
    z = np.load(os.path.join(GOLDEN, "indexer_small.npz"))
    case = {
        "b": 4, "s1": 2, "nh": 64, "d": 128, "block_size": 128, "selected_count": 64,
        "act_seq": z["act_seq"].tolist(), "query": torch.from_numpy(z["query"].copy()),
        "q_scale": _t16(z["q_scale"], torch.float16), "key_cache": torch.from_numpy(z["key_cache"].copy()),
        "k_scale": _t16(z["k_scale"], torch.float16), "weights": _t16(z["weights"], torch.float16),
        "block_table": torch.from_numpy(z["block_table"].copy()),
    }
    return case, torch.from_numpy(z["topk_res"].copy()), torch.from_numpy(z["scores_f64"].copy())
