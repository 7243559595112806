"""Random tiny configurations against the plain implementation: head sizes in steps of 16 up to
256 (and, listed by hand, head sizes and widths that the matrix-core kernels do not take), any
number of heads and groups, widths and vocabularies that are no power of two, two to five
layers in any arrangement of the two mixers, two to six taps with and without biases, tied and
untied heads. Each is stepped whole, in portions with single tokens between them, and as two
requests of which one decodes beside portions of the other, in float32 and in bfloat16."""

import tempfile

import numpy as np
import pytest

import plain_lfm2 as plain
from gpu_common import feed
from helpers import assert_close, random_tokens

pytestmark = pytest.mark.gpu


def random_config(rng) -> dict:
    head_dim = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256]))
    kv_heads = int(rng.choice([1, 2, 3]))
    heads = kv_heads * int(rng.choice([1, 2, 3, 4, 5, 8]))
    if heads * head_dim > 1536:         # keeps the plain implementation quick
        heads = max(kv_heads, (1536 // head_dim) // kv_heads * kv_heads)
    layers = int(rng.integers(2, 6))
    types = [str(rng.choice(["conv", "full_attention"])) for _ in range(layers)]
    for kind in ("conv", "full_attention"):
        if kind not in types:
            types[int(rng.integers(0, layers))] = kind
    return dict(
        architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=int(rng.choice([130, 257, 500, 1001])),
        hidden_size=heads * head_dim, num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=kv_heads,
        intermediate_size=int(rng.choice([72, 160, 200, 384])), block_auto_adjust_ff_dim=bool(rng.integers(0, 2)),
        block_ffn_dim_multiplier=float(rng.choice([1.0, 1.5])), block_multiple_of=int(rng.choice([8, 24, 64])),
        norm_eps=float(rng.choice([1e-5, 1e-6])), rope_theta=float(rng.choice([1e4, 1e6])),
        conv_L_cache=int(rng.integers(2, 7)), conv_bias=bool(rng.integers(0, 2)),
        tie_word_embeddings=bool(rng.integers(0, 2)), max_position_embeddings=512, layer_types=types)


def check_configuration(config: dict, seed: int, what: str) -> None:
    """One configuration against the plain model: whole, in portions, and as two requests of which
    one decodes beside portions of the other, in float32 and in bfloat16."""
    from flyweight_amd.config import config_from_dict
    from flyweight_amd.engine import StepEntry, Stepper, load_model
    from flyweight_amd.weights import write_random_model
    rng = np.random.default_rng(5000 + seed)
    with tempfile.TemporaryDirectory() as folder:
        write_random_model(folder, config_from_dict(config), seed=seed, scale="fan_in")
        plain_config, plain_weights = plain.read_folder(folder)
        tokens = random_tokens(config["vocab_size"], 140, seed=seed)
        other = random_tokens(config["vocab_size"], 75, seed=seed + 100)
        want, want_other = plain.forward(plain_config, plain_weights, tokens), plain.forward(plain_config, plain_weights, other)
        for dtype in ("float32", "bfloat16"):
            _, model = load_model(folder, dtype=dtype)
            stepper = Stepper(model, num_pages=6, max_requests=3)
            stepper.admit("r")
            assert_close(feed(stepper, "r", tokens, [140]), want, dtype, f"{what}: {dtype} whole")
            stepper.release("r")
            stepper.admit("r")
            cuts = [63, 2, 1, 1, 30, 1, 1, 1, 1, 1, 1, 1, 1, 20] + [1] * 20
            assert_close(feed(stepper, "r", tokens, cuts), want, dtype, f"{what}: {dtype} in portions")
            stepper.release("r")
            # two requests: "a" decodes token by token beside portions of one to eight tokens of "b"
            stepper.admit("a")
            stepper.admit("b")
            got_a = [stepper.step([StepEntry("a", tokens[:100], list(range(100)))]).cpu().numpy()]
            got_b, at_a, at_b = [], 100, 0
            while at_a < len(tokens) or at_b < len(other):
                entries, rows_a = [], 0
                if at_a < len(tokens):
                    entries.append(StepEntry("a", tokens[at_a:at_a + 1], [0]))
                    rows_a = 1
                portion = min(int(rng.integers(1, 9)), len(other) - at_b)
                if portion > 0:
                    entries.append(StepEntry("b", other[at_b:at_b + portion], list(range(portion))))
                out = stepper.step(entries).cpu().numpy()
                if rows_a:
                    got_a.append(out[:1])
                    at_a += 1
                if portion > 0:
                    got_b.append(out[rows_a:])
                    at_b += portion
            assert_close(np.concatenate(got_a), want, dtype, f"{what}: {dtype} decoding beside another's portions")
            assert_close(np.concatenate(got_b), want_other, dtype, f"{what}: {dtype} portions beside another's decoding")
            stepper.release("a")
            stepper.release("b")
            stepper.cache.check_invariants()
            assert stepper.cache.groups[0].pool.in_use == 0


@pytest.mark.parametrize("seed", range(12))
def test_a_random_configuration_matches_the_plain_model(seed):
    config = random_config(np.random.default_rng(1000 + seed))
    what = (f"head_dim {config['hidden_size'] // config['num_attention_heads']} heads {config['num_attention_heads']}/"
            f"{config['num_key_value_heads']} layers {config['layer_types']} taps {config['conv_L_cache']}")
    check_configuration(config, seed, what)


# Head sizes that are no multiple of 16 leave the matrix-core attention (bfloat16 too runs on the
# wave-per-row kernel, its rotation's partner lane half a head away where half is no power of
# two), widths that are no multiple of 8 leave the matrix-core products (rows of bfloat16 are
# then not 16-byte aligned), and a feed-forward width that is no multiple of 8 does the same to
# the product that reads it: (head size, heads, kv heads, feed-forward width).
ODD_SIZES = [(8, 4, 2, 72), (24, 3, 1, 100), (40, 2, 2, 160), (72, 2, 1, 52), (136, 2, 1, 200),
             (20, 3, 1, 90), (10, 5, 5, 36), (18, 3, 3, 70), (6, 6, 2, 44)]


@pytest.mark.parametrize("head_dim,heads,kv_heads,intermediate", ODD_SIZES)
def test_head_sizes_and_widths_that_the_matrix_core_kernels_do_not_take(head_dim, heads, kv_heads, intermediate):
    seed = head_dim
    rng = np.random.default_rng(seed)
    config = dict(
        architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=int(rng.choice([131, 257, 500])),
        hidden_size=heads * head_dim, num_hidden_layers=3, num_attention_heads=heads, num_key_value_heads=kv_heads,
        intermediate_size=intermediate, block_auto_adjust_ff_dim=False, norm_eps=float(rng.choice([1e-5, 1e-6])),
        rope_theta=float(rng.choice([1e4, 1e6])), conv_L_cache=int(rng.integers(2, 5)), conv_bias=bool(rng.integers(0, 2)),
        tie_word_embeddings=bool(rng.integers(0, 2)), max_position_embeddings=512,
        layer_types=["full_attention", "conv", "full_attention"])
    check_configuration(config, seed, f"head_dim {head_dim} heads {heads}/{kv_heads} hidden {heads * head_dim} ffn {intermediate}")


@pytest.mark.parametrize("hidden,heads,intermediate", [(2048, 32, 12288), (1024, 16, 6656)])
def test_a_wide_model_on_the_prompt_kernels(hidden, heads, intermediate):
    """The tiny models never reach the kernels that a real width selects for a prompt of 2,048
    tokens (256 x 256 and 256 x 192 tiles, the tiles of 128 or 64 columns whose waves split K,
    eight rows per thread in the row-wise kernels). Three layers of the 1.2B or the 350M shape's
    width with a small vocabulary do, and the plain model still takes seconds: one step of 2,048
    rows and 40 decoded tokens, then the same in portions that end inside pages, in bfloat16."""
    from flyweight_amd.config import config_from_dict
    from flyweight_amd.engine import Stepper, load_model
    from flyweight_amd.weights import write_random_model
    config = dict(
        architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=4096, hidden_size=hidden, num_hidden_layers=3,
        num_attention_heads=heads, num_key_value_heads=8, intermediate_size=intermediate, block_auto_adjust_ff_dim=True,
        block_ffn_dim_multiplier=1.0, block_multiple_of=256, norm_eps=1e-5, rope_theta=1000000.0, conv_L_cache=3,
        conv_bias=False, tie_word_embeddings=True, max_position_embeddings=4096,
        layer_types=["conv", "full_attention", "conv"])
    with tempfile.TemporaryDirectory() as folder:
        write_random_model(folder, config_from_dict(config), seed=1, scale="fan_in")
        plain_config, plain_weights = plain.read_folder(folder)
        tokens = random_tokens(config["vocab_size"], 2048 + 40, seed=3)
        want = plain.forward(plain_config, plain_weights, tokens)
        _, model = load_model(folder, dtype="bfloat16")
        stepper = Stepper(model, num_pages=40, max_requests=2)
        stepper.admit("r")
        assert_close(feed(stepper, "r", tokens, [2048] + [1] * 40), want, "bfloat16", "2,048 rows in one step, then 40 decoded")
        stepper.release("r")
        stepper.admit("r")
        assert_close(feed(stepper, "r", tokens, [1000, 1048, 40]), want, "bfloat16", "portions of 1,000, 1,048 and 40")
        stepper.release("r")
        stepper.cache.check_invariants()
