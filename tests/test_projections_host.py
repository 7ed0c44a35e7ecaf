"""Host side of the projection kernels: the RoPE parameters the library bakes into its launches
(`RopeScaling::kernel_parameters`, crates/inference-backend-metal/src/components/rms_norm_rope.rs:170-238)
against the reference's known answer and the oracle, and the config contract (rms_norm_rope.rs:81-96,154-168)."""
import ctypes

import numpy as np
import pytest


def yarn(psi, truncate=True):
    factor = float(np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0)))
    return psi.RopeScaling.Yarn(32.0, factor, 32.0, 1.0, 8192, truncate)


def test_yarn_correction_range_known_answer(psi):
    cfg = psi.RMSNormRopeConfig(1, 128, 128, 1e-6, 10_000_000.0, psi.Dtype.Float32, yarn(psi))
    inv, factor, corr = cfg.kernel_parameters()
    assert corr == (14.0, 29.0)
    assert factor == np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0))
    assert inv[0] == 1.0 and np.all(np.diff(inv) < 0)


@pytest.mark.parametrize("rope_dim,theta,scaling", [(2, 1e6, None), (64, 1e7, None), (128, 1e7, "yarn"),
                                                    (128, 1e7, "yarn-soft"), (256, 5e5, "yarn")])
def test_parameters_match_the_oracle_bit_for_bit(psi, oracle, rope_dim, theta, scaling):
    s = psi.RopeScaling() if scaling is None else yarn(psi, truncate=scaling == "yarn")
    cfg = psi.RMSNormRopeConfig(2, 256, rope_dim, 1e-6, theta, psi.Dtype.Bfloat16, s)
    inv, factor, corr = cfg.kernel_parameters()
    y = None if scaling is None else dict(factor=s.factor, attention_factor=s.attention_factor, beta_fast=s.beta_fast,
                                          beta_slow=s.beta_slow,
                                          original_max_position_embeddings=s.original_max_position_embeddings,
                                          truncate=s.truncate)
    o_inv, o_factor, o_corr = oracle.rope_parameters(rope_dim, theta, y)
    assert inv.view(np.uint32).tolist() == o_inv.view(np.uint32).tolist()
    assert factor == o_factor and corr == o_corr


@pytest.mark.parametrize("kwargs,text", [
    (dict(rope_dim=3), "rope_dim must be even"),
    (dict(rope_dim=0), "rope_dim must be even"),
    (dict(rope_dim=258, head_dim=256), "rope_dim must be even and in 2..head_dim"),
    (dict(eps=0.0), "eps must be finite and positive"),
    (dict(rope_theta=float("inf")), "rope_theta must be finite and positive"),
    (dict(rope_theta=1.0, yarn=True), "Yarn rope_theta must be greater than 1"),
    (dict(num_heads=0), "needs heads"),
])
def test_config_contract(psi, kwargs, text):
    base = dict(num_heads=2, head_dim=128, rope_dim=64, eps=1e-6, rope_theta=1e6)
    use_yarn = kwargs.pop("yarn", False)
    base.update(kwargs)
    cfg = psi.RMSNormRopeConfig(base["num_heads"], base["head_dim"], base["rope_dim"], base["eps"], base["rope_theta"],
                                psi.Dtype.Bfloat16, yarn(psi) if use_yarn else psi.RopeScaling())
    with pytest.raises(psi.PsiHipError) as err:
        cfg.kernel_parameters()
    assert text in str(err.value)


def test_yarn_scaling_contract(psi):
    bad = psi.RopeScaling.Yarn(0.5, 1.0, 32.0, 1.0, 8192, True)
    with pytest.raises(psi.PsiHipError) as err:
        psi.RMSNormRopeConfig(1, 128, 128, 1e-6, 1e7, psi.Dtype.Float32, bad).kernel_parameters()
    assert "Yarn factor" in str(err.value)
    swapped = psi.RopeScaling.Yarn(2.0, 1.0, 1.0, 32.0, 8192, True)
    with pytest.raises(psi.PsiHipError) as err:
        psi.RMSNormRopeConfig(1, 128, 128, 1e-6, 1e7, psi.Dtype.Float32, swapped).kernel_parameters()
    assert "beta_fast >= beta_slow" in str(err.value)
