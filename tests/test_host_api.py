"""Host-side behaviour that needs no GPU: the library loads and exports every symbol declared
in include/areal_hip.h, argument validation raises the reference's exception types before any
device work, and the product path refuses CPU tensors instead of falling back."""

import re
from pathlib import Path

import pytest
import torch

from areal_amd import _lib
from areal_amd.config import NormConfig, RejectionSamplingConfig
from areal_amd.data import KLEstimator, Normalization
from areal_amd.functional import (
    apply_rejection_sampling,
    cispo_loss_fn,
    fused_lm_head_logprobs_entropy,
    gather_logprobs,
    gather_logprobs_entropy,
    ppo_actor_loss_fn,
)
from areal_amd.functional.lm_head import default_token_chunk
from areal_amd.ppo.actor import grpo_loss_fn

ROOT = Path(__file__).resolve().parents[1]


def _declared_symbols():
    text = (ROOT / "include" / "areal_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(areal_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 17
    for name in names:
        assert hasattr(lib, name), f"{name} declared in areal_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names


def test_workspace_size_queries_run_without_gpu():
    lib = _lib.load()
    # H a multiple of 64 (hand-scheduled kernels, 2 slots per split): 4 vocabulary splits; the ragged
    # last vocabulary tile rides in the last split's sweep (a vocabulary that is not a multiple of 64
    # keeps a launch and a slot pair of its own). Other H (generic kernel): 4 slots per split
    assert lib.areal_lmhead_fwd_workspace_bytes(32768, 4096, 151936) == 7 * 8 * 32768 * 4
    assert lib.areal_lmhead_fwd_workspace_bytes(32768, 4096, 151936 - 8) == 7 * 10 * 32768 * 4
    assert lib.areal_lmhead_fwd_workspace_bytes(32768, 4096 + 64, 151936) == 7 * 8 * 32768 * 4
    assert lib.areal_lmhead_fwd_workspace_bytes(32768, 4096 + 8, 151936) == 7 * 16 * 32768 * 4
    # W^T [64, 1024] + dlogits [256, 1024]; a ragged chunk adds the two transposed copies
    assert lib.areal_lmhead_bwd_workspace_bytes(1024, 64, 1000, 256) >= 2 * (64 * 1024 + 256 * 1024)
    assert (lib.areal_lmhead_bwd_workspace_bytes(1000, 64, 1000, 256)
            > lib.areal_lmhead_bwd_workspace_bytes(1024, 64, 1000, 256) + 2 * 1000 * 256)
    # backward from saved exponentials: 594 x 16 dWeight tiles are 298 super-blocks of 32 workgroups,
    # 2 more than whole rounds of 8; those 384 vocabulary rows get fp32 partial results of 6 splits of
    # the token range (12 half-filled super-blocks, at most 32 workgroups on an XCD). 592 x 16 tiles are
    # whole rounds and need none.
    saved = lib.areal_lmhead_bwd_saved_workspace_bytes
    assert saved(32768, 4096, 151936) - saved(32768, 4096, 151552) == 6 * 384 * 4096 * 4 + 256
    # 144 x 2 tiles = 9 super-blocks: the last 16 tile columns (the test shape of tests/test_gpu_lmhead.py)
    assert saved(2048, 512, 36764) > 2 * (36764 - 128 * 256) * 512 * 4
    assert lib.areal_gae_workspace_bytes(0) == 0
    assert lib.areal_actor_loss_workspace_bytes(10, 3) > 0


def test_bf16_weight_gradient_needs_a_single_token_chunk():
    """areal_lmhead_bwd writes dWeight in bf16 itself (accumulate = 2) only when one token chunk
    covers the batch; the request is refused before anything is launched or read."""
    lib = _lib.load()
    fake = 0x10000  # never dereferenced: the argument checks come first
    args = [fake, fake, None, fake, fake, fake, fake, 512, 64, 1000, 1.0, 1.0, fake, fake, None]
    assert lib.areal_lmhead_bwd(*args, 2, 256, fake, 1 << 30, None) == _lib.ERR_UNSUPPORTED
    assert lib.areal_lmhead_bwd(*args, 3, 512, fake, 1 << 30, None) == -1  # bad argument


def test_no_cpu_fallback():
    h = torch.randn(4, 8).bfloat16()
    w = torch.randn(16, 8).bfloat16()
    y = torch.randint(0, 16, (4,))
    with pytest.raises(_lib.ArealHipError, match="no CPU fallback"):
        fused_lm_head_logprobs_entropy(h, w, y)
    with pytest.raises(_lib.ArealHipError, match="no CPU fallback"):
        gather_logprobs(torch.randn(4, 16), y)
    z = torch.zeros(4)
    with pytest.raises(_lib.ArealHipError, match="no CPU fallback"):
        ppo_actor_loss_fn(z, z, z, z, 0.2, torch.ones(4, dtype=torch.bool))
    with pytest.raises(_lib.ArealHipError, match="no CPU fallback"):
        Normalization(NormConfig())(z)


def test_lm_head_argument_errors():
    h = torch.randn(4, 8).bfloat16()
    w = torch.randn(16, 8).bfloat16()
    y = torch.randint(0, 16, (4,))
    with pytest.raises(ValueError, match="temperature must be positive"):
        fused_lm_head_logprobs_entropy(h, w, y, temperature=0.0)
    with pytest.raises(ValueError, match="temperature must be positive"):
        fused_lm_head_logprobs_entropy(h, w, y, temperature=float("nan"))
    with pytest.raises(ValueError, match="logit_scale must be positive"):
        fused_lm_head_logprobs_entropy(h, w, y, logit_scale=-1.0)
    with pytest.raises(ValueError, match="chunk_size must be positive"):
        fused_lm_head_logprobs_entropy(h, w, y, token_chunk=0)
    with pytest.raises(ValueError, match="matching hidden and weight dtypes"):
        fused_lm_head_logprobs_entropy(h.float(), w, y)
    with pytest.raises(ValueError, match="leading dimensions must match labels"):
        fused_lm_head_logprobs_entropy(h, w, y[:3])
    assert default_token_chunk(32768, 4096, 151936) == 32768
    assert default_token_chunk(131072, 5120, 151936) % 256 == 0


def test_logits_argument_errors():
    with pytest.raises(ValueError, match="temperature must be positive"):
        gather_logprobs_entropy(torch.randn(4, 16), torch.zeros(4, dtype=torch.long), temperature=-1.0)
    with pytest.raises(ValueError, match="leading dimensions must match labels"):
        gather_logprobs(torch.randn(4, 16), torch.zeros(3, dtype=torch.long))


def test_loss_argument_errors():
    z = torch.zeros(4)
    m = torch.ones(4, dtype=torch.bool)
    # messages matched by the reference's tests (tests/test_functional.py:665,762)
    with pytest.raises(ValueError, match="cu_seqlens is required"):
        ppo_actor_loss_fn(z, z, z, z, 0.2, m, importance_sampling_level="sequence")
    with pytest.raises(ValueError, match="Invalid importance_sampling_level"):
        ppo_actor_loss_fn(z, z, z, z, 0.2, m, importance_sampling_level="invalid")
    with pytest.raises(AssertionError):
        ppo_actor_loss_fn(z, z, z, z, 0.2, m, c_clip=1.0)
    for bad in (None, 0.0, -1.0):  # tests/test_cispo_loss.py:96-108
        with pytest.raises(ValueError, match="eps_clip_higher"):
            cispo_loss_fn(z, z, z, 1.0, m, eps_clip_higher=bad)
    cfg = RejectionSamplingConfig(level="token", metric="ratio", upper=5.0)
    with pytest.raises(ValueError, match="shape"):  # tests/test_rejection_sampling.py:796-810
        apply_rejection_sampling(torch.zeros(1, 2), torch.zeros(1, 3), torch.ones(1, 2), None, cfg)
    seq = RejectionSamplingConfig(level="sequence", metric="ratio", upper=5.0)
    with pytest.raises(ValueError, match="cu_seqlens is required"):
        apply_rejection_sampling(z, z, torch.ones(4), None, seq)
    with pytest.raises(ValueError, match="ndim"):
        apply_rejection_sampling(torch.zeros(1, 1, 2), torch.zeros(1, 1, 2), torch.ones(1, 1, 2), None, cfg)


def test_rejection_sampling_config_validation():
    # tests/test_rejection_sampling.py:813-839 and :24-42
    with pytest.raises(ValueError, match="lower.*cannot be greater than upper"):
        RejectionSamplingConfig(metric="ratio", lower=3.0, upper=2.0)
    for field in ("level", "action", "metric", "agg"):
        with pytest.raises(ValueError, match=f"{field} must be one of"):
            RejectionSamplingConfig(**{field: "invalid"})
    with pytest.raises(ValueError, match="upper must be > 1.0"):
        RejectionSamplingConfig(metric="ratio", upper=1.0)
    with pytest.raises(ValueError, match="lower must be positive"):
        RejectionSamplingConfig(metric="ratio", lower=0.0, upper=2.0)
    with pytest.raises(ValueError, match="only supports metric='ratio'"):
        RejectionSamplingConfig(action="clamp", metric="kl_k2", upper=1.0)
    assert RejectionSamplingConfig(action="clamp", metric="ratio", upper=5.0).lower == 0.0
    with pytest.warns(UserWarning, match="ignored when level='token'"):
        RejectionSamplingConfig(level="token", agg="max")
    assert RejectionSamplingConfig(metric="binary_kl", upper=0.05).metric == "binary_kl"


def test_norm_config_and_group_errors():
    with pytest.raises(ValueError, match="mean_level"):
        NormConfig(mean_level="token")
    with pytest.raises(ValueError, match="group_size must be a positive integer"):
        NormConfig(mean_level="group", group_size=0)
    norm = Normalization(NormConfig(mean_level="group", std_level="group", group_size=2))
    with pytest.raises(ValueError, match="must equal"):
        norm._group_rows(4, [3, 2])
    with pytest.raises(ValueError, match="positive"):
        norm._group_rows(4, [4, 0])
    assert norm._group_rows(5, None) == ((2, 2), 1)
    assert norm._group_rows(8, [3, 2, 3]) == ((3, 2, 3), 0)


def test_kl_estimator_values():
    a, b = torch.tensor([0.5, -0.5, 20.0]), torch.zeros(3)
    assert torch.equal(KLEstimator("k1")(a, b), torch.tensor([0.5, -0.5, 10.0]))
    torch.testing.assert_close(KLEstimator("k2", apply_clamp=False)(a, b), a * a / 2)
    torch.testing.assert_close(KLEstimator("k3", apply_clamp=False)(a, b), torch.exp(-a) - 1 + a)
    with pytest.raises(ValueError, match="Invalid KL estimator"):
        KLEstimator("k4")


def test_grpo_loss_fn_rejects_out_of_scope_options():
    z = torch.zeros(4)
    data = dict(logprobs=z, advantages=z, loss_mask=torch.ones(4), prox_logp=z)
    with pytest.raises(ValueError, match="not compatible with `use_decoupled_loss=True`"):
        grpo_loss_fn(z, z, data, 0.2, None, None, use_sapo_loss=True, use_decoupled_loss=True)
    with pytest.raises(ValueError, match="not a valid ProxLogpMethod"):
        grpo_loss_fn(z, z, data, 0.2, None, None, prox_logp_method="guess")
    with pytest.raises(ValueError, match="versions not available"):
        grpo_loss_fn(z, z, dict(data, prox_logp=None), 0.2, None, None, prox_logp_method="loglinear")
    with pytest.raises(ValueError, match="mutually exclusive"):
        grpo_loss_fn(z, z, data, 0.2, 4.0, None, use_cispo_loss=True, use_sapo_loss=True)
    with pytest.raises(ValueError, match="CISPO only supports"):
        grpo_loss_fn(z, z, data, 0.2, 4.0, None, use_cispo_loss=True, importance_sampling_level="sequence")
    data["prox_logp"] = None
    with pytest.raises(ValueError, match="prox_logp is None"):
        grpo_loss_fn(z, z, data, 0.2, None, None)
    data["prox_logp"] = torch.tensor([0.0, float("nan"), 0.0, 0.0])
    with pytest.raises(RuntimeError, match="NaN or Inf"):
        grpo_loss_fn(z, z, data, 0.2, None, None)


def _length_context(lengths):
    return {"effective_token_lengths": lengths, "turn_counts": lengths, "timestep_lengths": lengths}


def test_gae_lambda_schedules_reference_literals():
    # the values the reference's tests pin for areal/trainer/ppo/lambda_fn.py
    # (tests/test_ppo_gae.py:279-341 VAPO, :344-390 relative position), on the package's functions
    from areal_amd.ppo.lambda_fn import (
        constant_gae_lambda,
        relative_position_gae_lambda,
        vapo_length_adaptive_gae,
    )

    q = 0.3
    lengths = torch.tensor([10, 19])
    lam = relative_position_gae_lambda(_length_context(lengths), q=q)
    assert lam.dtype == torch.float32
    torch.testing.assert_close(lam.pow((lengths - 1).float()), torch.full((2,), q), rtol=1e-6, atol=1e-7)
    # step 5 of 10 and step 9 of 19 are both at relative position 4 / 9
    torch.testing.assert_close(lam.pow(torch.tensor([5.0, 10.0])), torch.full((2,), q ** (5.0 / 9.0)), rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(relative_position_gae_lambda(_length_context(torch.tensor([0, 1, 2])), q=0.3),
                               torch.tensor([0.0, 1.0, 0.3]), rtol=0.0, atol=1e-7)
    assert torch.equal(relative_position_gae_lambda(_length_context(torch.tensor([0, 1, 5])), q=1),
                       torch.tensor([0.0, 1.0, 1.0]))
    assert torch.equal(vapo_length_adaptive_gae(_length_context(torch.tensor([4, 2, 0])), alpha=1.0),
                       torch.tensor([0.75, 0.5, 0.0]))
    # short trajectories: 1 - 1 / (alpha L) < 0 is floored at 0
    torch.testing.assert_close(vapo_length_adaptive_gae(_length_context(torch.tensor([1, 2, 3, 8])), alpha=0.5),
                               torch.tensor([0.0, 0.0, 1.0 - 1.0 / 1.5, 0.75]), rtol=1e-6, atol=1e-7)
    lam = constant_gae_lambda(_length_context(torch.tensor([3, 0, 7])), value=0.95)
    assert lam.dtype == torch.float32 and torch.equal(lam, torch.full((3,), 0.95))


@pytest.mark.parametrize("q", [True, -0.1, 0.0, 1.1, float("nan"), float("inf"), "0.5", None])
def test_relative_position_gae_lambda_rejects_invalid_q(q):
    # tests/test_ppo_gae.py:392-403
    from areal_amd.ppo.lambda_fn import relative_position_gae_lambda

    with pytest.raises(ValueError, match=r"q must be .* in \(0, 1\]"):
        relative_position_gae_lambda(_length_context(torch.tensor([2])), q=q)


@pytest.mark.parametrize("alpha", [0.0, -1.0, True, "1", None, float("nan")])
def test_vapo_gae_lambda_rejects_non_positive_alpha(alpha):
    # tests/test_ppo_gae.py:499-508: checked even when every trajectory is empty
    from areal_amd.ppo.lambda_fn import vapo_length_adaptive_gae

    with pytest.raises(ValueError, match="alpha must be a positive number"):
        vapo_length_adaptive_gae(_length_context(torch.tensor([0])), alpha=alpha)


def test_resolve_gae_lambda_fn():
    # areal/trainer/ppo/lambda_fn.py:115-141: a number -> the constant schedule (not custom), a
    # dotted path -> the imported callable (custom), anything else -> TypeError
    from areal_amd.ppo import lambda_fn as LF

    fn, custom = LF.resolve_gae_lambda_fn(0.9)
    assert custom is False
    assert torch.equal(fn(_length_context(torch.tensor([5, 0]))), torch.full((2,), 0.9))
    fn, custom = LF.resolve_gae_lambda_fn(1)
    assert custom is False and torch.equal(fn(_length_context(torch.tensor([2]))), torch.ones(1))
    fn, custom = LF.resolve_gae_lambda_fn("areal_amd.ppo.lambda_fn.vapo_length_adaptive_gae")
    assert custom is True and fn is LF.vapo_length_adaptive_gae
    with pytest.raises(TypeError, match="not bool"):
        LF.resolve_gae_lambda_fn(True)
    for bad in ("", None, [0.9]):
        with pytest.raises(TypeError, match="float or a non-empty dotted function path"):
            LF.resolve_gae_lambda_fn(bad)
    with pytest.raises(TypeError, match="not callable"):
        LF.resolve_gae_lambda_fn("areal_amd.ppo.lambda_fn.__all__")
    with pytest.raises(ValueError, match="Invalid module path"):
        LF.resolve_gae_lambda_fn("no_dots")
    with pytest.raises(ImportError, match="Failed to import module"):
        LF.resolve_gae_lambda_fn("areal_amd.no_such_module.fn")
    with pytest.raises(AttributeError, match="has no attribute"):
        LF.resolve_gae_lambda_fn("areal_amd.ppo.lambda_fn.no_such_fn")


def test_reward_overlong_penalty_matches_the_reference_loop():
    # areal/utils/functional/functional.py:937-959 restated as its per-sample loop (the
    # reference has no test for it); the vector form must give the same rewards, in place.
    from areal_amd.functional import reward_overlong_penalty

    loss_mask = torch.zeros(5, 40)
    for i, n in enumerate([10, 24, 30, 36, 40]):
        loss_mask[i, :n] = 1
    rewards = torch.tensor([1.0, 0.0, 1.0, 1.0, 0.5])
    data = dict(rewards=rewards.clone(), loss_mask=loss_mask, input_ids=torch.zeros(5, 40, dtype=torch.long))
    held = data["rewards"]
    out = reward_overlong_penalty(data, overlong_tokens=8, overlong_penalty_factor=1.5, max_response_length=32)
    want = rewards.clone()
    for i, n in enumerate([10, 24, 30, 36, 40]):
        want[i] += min(-(n - (32 - 8)) / 8 * 1.5, 0)
    assert out is data and data["rewards"] is held  # updated in place
    torch.testing.assert_close(data["rewards"], want)
    assert data["rewards"].tolist() == pytest.approx([1.0, 0.0, -0.125, -1.25, -2.5])


def test_chunked_lm_head_wrapper_refuses_what_the_reference_refuses():
    # vocab_parallel_head.py:953-966: same exception types and messages; the bias is taken from
    # the layer unless skip_bias_add
    from types import SimpleNamespace

    from areal_amd.functional import chunked_lm_head_logprobs_entropy as head

    h, w, y = torch.zeros(4, 8, dtype=torch.bfloat16), torch.zeros(16, 8, dtype=torch.bfloat16), torch.zeros(4, dtype=torch.long)
    ok = SimpleNamespace(bias=None, skip_bias_add=False, gather_output=False, tp_group=None,
                         config=SimpleNamespace(defer_embedding_wgrad_compute=False))
    with pytest.raises(NotImplementedError, match="forward override"):
        head(SimpleNamespace(chunked_loss_supported=False), h, w, y, temperature=1.0, chunk_size=4)
    with pytest.raises(NotImplementedError, match="defer_embedding_wgrad_compute"):
        head(SimpleNamespace(config=SimpleNamespace(defer_embedding_wgrad_compute=True)), h, w, y,
             temperature=1.0, chunk_size=4)
    with pytest.raises(NotImplementedError, match="ungathered"):
        head(SimpleNamespace(gather_output=True), h, w, y, temperature=1.0, chunk_size=4)
    with pytest.raises(ValueError, match="chunk_size must be positive"):
        head(ok, h, w, y, temperature=1.0, chunk_size=0)
    with pytest.raises(ValueError, match="temperature must be positive"):
        head(ok, h, w, y, temperature=0.0, chunk_size=4)
    with pytest.raises(_lib.ArealHipError):  # valid arguments reach the kernels, which need the GPU
        head(ok, h, w, y, temperature=1.0, chunk_size=4)

