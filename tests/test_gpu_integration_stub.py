"""The ctypes stub printed in the integration notes at the repository root, executed as it stands:
the python block under "Binding the C ABI directly" binds one entry point and must give the
oracle's log-probs and entropies."""
import os
import re

import pytest
import torch

from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def test_the_documented_stub_runs(cuda):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    section = text[text.index("## 3. Binding the C ABI directly"):]
    block = re.search(r"```python\n(.*?)```", section, re.S).group(1)
    scope = {}
    cwd = os.getcwd()
    os.chdir(root)  # the stub opens the library by its path relative to the repository root
    try:
        exec(compile(block, "<documented stub>", "exec"), scope)
        g = torch.Generator().manual_seed(0)
        x = (torch.randn(300, 4099, generator=g) * 2).to(torch.bfloat16)
        labels = torch.randint(0, 4099, (300,), generator=g)
        lp, ent, stats = scope["fused_logprob_entropy"](x.to(cuda), labels.to(cuda), 0.8)
        torch.cuda.synchronize()
    finally:
        os.chdir(cwd)
    assert (lp.cpu().double() - otn.log_probs_from_logits(x.double(), labels, 0.8)).abs().max().item() <= 2e-3
    assert (ent.cpu().double() - otn.compute_entropy(x.double())).abs().max().item() <= 2e-3
    assert stats.shape == (300, 4)
