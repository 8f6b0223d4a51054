"""The drop-in boundary is the reference's Python signatures: argument names, order, defaults.

The reference's source files are parsed as text (never imported) where they are present; the
test is skipped elsewhere."""

import ast
import inspect
import os

import pytest

REF = "/root/reference/areal"

CASES = [
    ("utils/functional/functional.py", "areal_amd.functional",
     ["apply_rejection_sampling", "cispo_loss_fn", "dpo_pair_logratios", "dpo_preference_loss",
      "masked_normalization", "ppo_actor_loss_fn", "ppo_critic_loss_fn", "reward_overlong_penalty",
      "sapo_loss_fn"]),
    ("utils/functional/vocab_parallel.py", "areal_amd.functional", ["gather_logprobs", "gather_logprobs_entropy"]),
    ("trainer/ppo/actor.py", "areal_amd.ppo.actor", ["grpo_loss_fn", "compute_prox_logp_approximations"]),
    ("trainer/ppo/gae.py", "areal_amd.ppo.gae",
     ["_compute_token_level_gae", "_compute_turn_level_gae", "_build_gae_lambda_context"]),
    ("trainer/ppo/lambda_fn.py", "areal_amd.ppo.lambda_fn",
     ["constant_gae_lambda", "vapo_length_adaptive_gae", "relative_position_gae_lambda", "resolve_gae_lambda_fn"]),
]


def _reference_signatures(path, names):
    tree = ast.parse(open(path).read())
    out = {}
    for node in tree.body:  # module-level functions only
        if isinstance(node, ast.FunctionDef) and node.name in names:
            a = node.args
            pos = [x.arg for x in a.posonlyargs + a.args]
            n_def = len(a.defaults)
            defaults = dict(zip(pos[len(pos) - n_def:], (ast.unparse(d) for d in a.defaults)))
            kwonly = [x.arg for x in a.kwonlyargs]
            kwdefaults = {k.arg: ast.unparse(d) for k, d in zip(a.kwonlyargs, a.kw_defaults) if d is not None}
            out[node.name] = (pos, defaults, kwonly, kwdefaults)
    return out


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference sources are not present here")
@pytest.mark.parametrize("rel,module,names", CASES, ids=[c[0] for c in CASES])
def test_signatures(rel, module, names):
    import importlib

    mod = importlib.import_module(module)
    ref = _reference_signatures(os.path.join(REF, rel), names)
    for name in names:
        assert name in ref, f"{name} not found in the reference's {rel}"
        rpos, rdef, rkw, rkwdef = ref[name]
        params = inspect.signature(getattr(mod, name)).parameters.values()
        pos = [p.name for p in params if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
        kw = [p.name for p in params if p.kind == p.KEYWORD_ONLY]
        # ours may append keyword arguments of its own after the reference's
        assert pos[: len(rpos)] == rpos, (name, pos, rpos)
        assert [k for k in kw if k in rkw] == rkw, (name, kw, rkw)
        for p in params:
            want = rdef.get(p.name, rkwdef.get(p.name))
            if want is None or p.default is p.empty:
                continue
            try:
                want_value = ast.literal_eval(want)
            except (ValueError, SyntaxError):
                continue  # a named constant or call: compared by the tests of that function
            assert p.default == want_value, (name, p.name, p.default, want)


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference sources are not present here")
@pytest.mark.parametrize("name", ["NormConfig", "RejectionSamplingConfig"])
def test_config_dataclass_fields(name):
    import dataclasses

    from areal_amd import config

    tree = ast.parse(open(os.path.join(REF, "api/cli_args.py")).read())
    node = next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == name)
    want = []
    for st in node.body:
        if not (isinstance(st, ast.AnnAssign) and isinstance(st.target, ast.Name)):
            continue
        default = None
        if isinstance(st.value, ast.Call) and getattr(st.value.func, "id", None) == "field":
            for k in st.value.keywords:
                if k.arg == "default":
                    default = ast.literal_eval(k.value)
        elif st.value is not None:
            default = ast.literal_eval(st.value)
        want.append((st.target.id, default))
    got = [(f.name, None if f.default is dataclasses.MISSING else f.default)
           for f in dataclasses.fields(getattr(config, name))]
    assert got == want

