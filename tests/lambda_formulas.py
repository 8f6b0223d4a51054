"""Per-trajectory GAE lambda schedules used by the tests (test helpers, not product code).

``compute_advantages(gae_lambda_fn=...)`` accepts any callable ``fn(context, **kwargs)`` that
maps the length context of ``_build_gae_lambda_context`` to one lambda per trajectory; the
reference ships such callables in ``areal/trainer/ppo/lambda_fn.py:37-112`` and they work with
this package unchanged (plain torch on ``[bs]`` tensors).  The two schedules below are written
from their published closed forms so that the tests do not depend on the reference being
importable:

* VAPO length-adaptive:  lambda = max(0, 1 - 1 / (alpha * L)), and 0 for L = 0;
* relative position:     lambda = q^(1 / (L - 1)) for L >= 2, 1 for L = 1, 0 for L = 0.
"""

import torch


def vapo(context, *, alpha):
    n = context["timestep_lengths"]
    lam = torch.zeros(n.shape, dtype=torch.float32, device=n.device)
    pos = n > 0
    lam[pos] = torch.clamp(1.0 - 1.0 / (alpha * n[pos].float()), min=0.0)
    return lam


def relative_position(context, *, q):
    n = context["timestep_lengths"]
    lam = torch.zeros(n.shape, dtype=torch.float32, device=n.device)
    lam[n == 1] = 1.0
    many = n >= 2
    lam[many] = torch.tensor(float(q), device=n.device) ** (1.0 / (n[many] - 1).float())
    return lam
