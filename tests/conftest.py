import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=64, n_head=4,
              n_inner=256, vocab_size=512, n_positions=128, layer_norm_epsilon=1e-5,
              activation_function="gelu_new", scale_attn_by_inverse_layer_idx=False)
TINY_B = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=3, n_embd=96, n_head=2,
              n_inner=320, vocab_size=1000, n_positions=256, layer_norm_epsilon=1e-6,
              activation_function="gelu", scale_attn_by_inverse_layer_idx=True)
# a third, for long sequences and other head sizes: 3 heads of 32, odd vocabulary
TINY_C = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=96, n_head=3,
              n_inner=200, vocab_size=777, n_positions=640, layer_norm_epsilon=1e-5,
              activation_function="gelu_new", scale_attn_weights=True)
# a fourth with the head size and context of the large models (4 heads of 64, 1024 positions)
TINY_D = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=256, n_head=4,
              vocab_size=5003, n_positions=1024, layer_norm_epsilon=1e-5, activation_function="gelu_new")
# a fifth, one wide layer: its products have the widths (more than 4,096 columns) at which steps of
# 129 to 256 rows change kernels
WIDE_E = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=1, n_embd=1408, n_head=22,
              vocab_size=300, n_positions=64, layer_norm_epsilon=1e-5, activation_function="gelu_new")
# a sixth, two layers of 1,024 columns: the least width at which steps of 17 to 64 rows run their norms
# inside the products beside them, across the blocks' border too
WIDE_F = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=1024, n_head=16,
              vocab_size=300, n_positions=64, layer_norm_epsilon=1e-5, activation_function="gelu")
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3), "E": (WIDE_E, 4), "F": (WIDE_F, 5)}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a GPU (run on the MI355X box)")


@pytest.fixture(autouse=True)
def _seeded(request):
    """Every test starts from the same state of torch's default generators (CPU and device), derived from its
    name, so that a test that draws without a generator of its own draws the same numbers in every run."""
    import zlib
    torch.manual_seed(zlib.crc32(request.node.nodeid.encode()))


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """{(name, storage dtype): folder} of random-weight model folders, made on demand."""
    from denno_beta_amd.weights import write_model_folder
    made = {}

    def get(name, dtype="float32"):
        key = (name, dtype)
        if key not in made:
            cfg, seed = TINY[name]
            d = tmp_path_factory.mktemp(f"tiny{name}_{dtype}")
            write_model_folder(str(d), cfg, seed, dtype)
            made[key] = str(d)
        return made[key]
    return get


def seeded_tokens(seed, n, vocab):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


BACKENDS = [pytest.param("host", id="host"), pytest.param("gpu", marks=pytest.mark.gpu, id="gpu")]


@pytest.fixture(params=BACKENDS)
def backend(request):
    """The device the engine runs on.  "gpu": the HIP kernels.  "host": the same engine code on
    the CPU with the kernels' plain references in their place, so that cache, batch and
    scheduling logic is tested where there is no GPU."""
    if request.param == "host":
        from emulation import emulated_kernels
        with emulated_kernels():
            yield "cpu"
    else:
        yield "cuda:0"
