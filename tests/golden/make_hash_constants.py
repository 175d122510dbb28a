"""Regenerates tests/golden/hash_constants.json: the eight hash constants per seed, drawn with
plain torch exactly as the reference module draws them (python/rz_linear/RzLinear.py:68-74:
torch.manual_seed(seed); torch.randint(0, P, (R-1,)); P prepended).  Runs no reference code."""
import json
import os

import torch

P, R = 45007, 8
out = {"P": P, "seeds": {}}
for seed in (1024, 0, 1, 42):
    torch.manual_seed(seed)
    out["seeds"][str(seed)] = [P] + torch.randint(0, P, (R - 1,)).tolist()
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hash_constants.json")
old = json.load(open(path)) if os.path.exists(path) else {}
out["_comment"] = old.get("_comment", "")
json.dump(out, open(path, "w"), indent=2)
print(out)
