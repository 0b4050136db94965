import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "inferred-thoughts_amd"))
sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return ROOT / "tests" / "golden"


@pytest.fixture(scope="session")
def tiny_gguf(tmp_path_factory):
    """Config 1 of the baseline: tiny hybrid MoE, all Q8_0, seed 0."""
    import inferred_hip as ih
    p = tmp_path_factory.mktemp("models") / "tiny_q8_0.gguf"
    ih.synth_write_gguf(str(p), ih.tiny_config(seed=0))
    return p


@pytest.fixture(scope="session")
def mid_gguf(tmp_path_factory):
    """Config 5's layer shapes and formats (hidden 2048, NVFP4 experts of 512, head_dim 256, dk = dv = 128,
    top-10 routing) cut down to 4 layers, 32 experts and a vocabulary of 8192: about 0.4 GB."""
    import inferred_hip as ih
    p = tmp_path_factory.mktemp("models") / "mid_nvfp4.gguf"
    ih.synth_write_gguf(str(p), ih.big_config(seed=2, n_layer=4, n_vocab=8192, n_expert=32, n_threads=8))
    return p


@pytest.fixture(scope="session")
def tiny_f32_router_gguf(tmp_path_factory):
    """The tiny shape with the router, the shared-expert gate and ssm alpha / beta in F32, as real files keep them
    (the matrices that decide which experts run), and NVFP4 experts."""
    import inferred_hip as ih
    p = tmp_path_factory.mktemp("models") / "tiny_f32_router.gguf"
    ih.synth_write_gguf(str(p), ih.tiny_config(seed=3, expert_type=ih.NVFP4, router_type=ih.ROUTER_F32))
    return p


@pytest.fixture(scope="session")
def tiny_nvfp4_gguf(tmp_path_factory):
    """The tiny shape with NVFP4 experts and per-expert scales (exercises config 5's formats)."""
    import inferred_hip as ih
    p = tmp_path_factory.mktemp("models") / "tiny_nvfp4.gguf"
    ih.synth_write_gguf(str(p), ih.tiny_config(seed=1, expert_type=ih.NVFP4))
    return p


@pytest.fixture(scope="session")
def tiny_real_layout_gguf(tmp_path_factory):
    """The tiny shape laid out as an NVFP4 file of this model is: NVFP4 experts with per-expert scales, an NVFP4 shared
    expert with a second scale per matrix (ffn_*_shexp.scale), and the router, shared-expert gate and ssm alpha / beta
    in F32."""
    import inferred_hip as ih
    p = tmp_path_factory.mktemp("models") / "tiny_real_layout.gguf"
    ih.synth_write_gguf(str(p), ih.tiny_config(seed=4, expert_type=ih.NVFP4, shared_type=ih.NVFP4, router_type=ih.ROUTER_F32))
    return p


@pytest.fixture(scope="session")
def tiny_nvfp4_shared_gguf(tmp_path_factory):
    """The tiny shape with NVFP4 experts and an NVFP4 shared expert with second scales, Q8_0 router (so that exact mode
    fuses the routed FFN of a single-token pass as well)."""
    import inferred_hip as ih
    p = tmp_path_factory.mktemp("models") / "tiny_nvfp4_shared.gguf"
    ih.synth_write_gguf(str(p), ih.tiny_config(seed=5, expert_type=ih.NVFP4, shared_type=ih.NVFP4))
    return p
