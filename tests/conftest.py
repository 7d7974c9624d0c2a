import json
import os
import sys
import types

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_known_answers.json")) as f:
        return json.load(f)


def make_grpo_config(**overrides):
    """Duck-typed stand-in for GRPOExperimentConfig with the defaults of the reference's own test
    helper (open_instruct/test_olmo_core_train_modules.py:155-175)."""
    cfg = dict(
        clip_lower=0.2, clip_higher=0.2, beta=0.05, kl_estimator=2, loss_fn="dapo", load_ref_policy=False,
        rho_mask_sequence_level=False, rho_clamp_lower_bound=0.0, rho_clamp_upper_bound=0.0,
        rho_mask_lower_bound=0.0, rho_mask_upper_bound=0.0, rho_mask_tv_divergence=False, use_rho_correction=False,
    )  # fmt: skip
    cfg.update(overrides)
    return types.SimpleNamespace(**cfg)


@pytest.fixture
def grpo_config():
    return make_grpo_config
