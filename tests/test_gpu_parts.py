"""Each part of a layer alone, built from its PartSpec with its own sizes, against the
plain implementation's function for that part; and toy parts defined here (a mixer with state
of its own kind that does not start at zero, a feed-forward with routing, another position
encoding) that are registered, built and stepped without touching the framework."""

import dataclasses
import math
import os

import numpy as np
import pytest
import torch

import plain_lfm2 as plain

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 5e-6, torch.bfloat16: 2e-2}


def close(found, expected, dtype):
    found = found.detach().cpu().double().numpy()
    limit = TOL[dtype] * max(1.0, float(np.abs(expected).max()))
    assert found.shape == expected.shape and np.isfinite(found).all()
    assert float(np.abs(found - expected).max()) <= limit, f"{float(np.abs(found - expected).max()):.3e} > {limit:.3e}"


def bound(part, dtype, seed=0):
    """Random tensors for a part, bound on the GPU; returns them as float64 numpy too."""
    from flyweight_amd.weights import random_tensors
    from flyweight_amd.weights.loader import storage_dtype
    tensors = random_tensors(part.tensors(), seed, torch.bfloat16, scale="fan_in")
    device = {n: t.to(storage_dtype(part.tensors()[n].role, t.dtype, dtype)).to(DEV) for n, t in tensors.items()}
    part.bind(device, dtype, DEV)
    return {n: t.double().numpy() for n, t in tensors.items()}




class Harness:
    """A cache for one mixer and step contexts over it."""

    def __init__(self, mixer, dtype, num_pages=8, max_requests=4):
        from flyweight_amd.cache import CacheManager
        need = mixer.cache_need()
        self.cache = CacheManager({0: need} if need is not None else {}, num_pages=num_pages, max_requests=max_requests,
                                  dtype=dtype, device=DEV)
        self.mixer = mixer

    def run(self, entries, h):
        """entries: [(request, count)]; h: [rows, hidden] on the device. Returns the mixer's
        contribution to the residual."""
        from flyweight_amd.config import ScheduleEntry
        from flyweight_amd.engine.step import StepContext, StepEntry
        step = []
        for request, count in entries:
            if request not in self.cache.requests:
                self.cache.admit(request)
            self.cache.reserve(request, self.cache.length_of(request) + count)
            step.append(StepEntry(request, [0] * count, []))
        ctx = StepContext(step, self.cache, DEV, vocab_size=1, max_positions=1 << 20)
        residual = torch.zeros(h.shape[0], self.mixer.hidden, dtype=torch.float32, device=DEV)
        self.mixer.forward(h, residual, ctx, ctx.cache_view(self.cache, ScheduleEntry(0, cache=0)))
        for request, length in zip(ctx.requests, ctx.new_lengths):
            self.cache.commit(request, length)
        return residual


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from flyweight_amd.config import PartSpec
    from flyweight_amd.parts import build_part
    part = build_part("norm", PartSpec("rmsnorm", {"size": 100, "eps": 3e-4}, prefix="n."))
    w = bound(part, dtype)
    x = torch.randn(6, 100, generator=torch.Generator().manual_seed(1)) * 2
    close(part.forward(x.to(DEV), None), plain.rms_norm(x.double().numpy(), w["n.weight"], 3e-4), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part(dtype):
    from flyweight_amd.config import PartSpec
    from flyweight_amd.parts import build_part
    part = build_part("ffn", PartSpec("swiglu", {"hidden_size": 72, "intermediate_size": 200,
                                                 "names": {"gate": "w1", "up": "w3", "down": "w2"}}, prefix="f."))
    w = bound(part, dtype)
    h = (torch.randn(9, 72, generator=torch.Generator().manual_seed(2))).to(dtype)
    residual = torch.ones(9, 72, dtype=torch.float32, device=DEV)
    part.forward(h.to(DEV), residual, None)
    close(residual, 1.0 + plain.swiglu(h.double().numpy(), w, "f."), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,kernel,bias", [(72, 3, False), (40, 5, True)])
def test_short_conv_part_whole_and_cut(dtype, hidden, kernel, bias):
    from flyweight_amd.config import PartSpec
    from flyweight_amd.parts import build_part
    part = build_part("mixer", PartSpec("short_conv", {"hidden_size": hidden, "kernel_size": kernel, "bias": bias}, prefix="c."))
    w = bound(part, dtype, seed=3)
    T = 50
    h = torch.randn(T, hidden, generator=torch.Generator().manual_seed(4)).to(dtype)
    want = plain.short_conv_mixer(h.double().numpy(), w, "c.", {"hidden_size": hidden, "conv_bias": bias})
    harness = Harness(part, dtype)
    close(harness.run([("whole", T)], h.to(DEV)), want, dtype)
    pieces, at = [], 0
    for n in (3, 1, 2, 20, 1, 1, 22):       # portions shorter than the kernel's reach too
        pieces.append(harness.run([("cut", n)], h[at:at + n].contiguous().to(DEV)))
        at += n
    close(torch.cat(pieces), want, dtype)
    # two sequences in one batch, one decoding while the other is in a portion
    other = torch.randn(8, hidden, generator=torch.Generator().manual_seed(5)).to(dtype)
    want_other = plain.short_conv_mixer(other.double().numpy(), w, "c.", {"hidden_size": hidden, "conv_bias": bias})
    first = harness.run([("x", 7), ("y", 5)], torch.cat([other[:7], h[:5]]).to(DEV))
    second = harness.run([("y", 3), ("x", 1)], torch.cat([h[5:8], other[7:8]]).to(DEV))
    close(torch.cat([first[:7], second[3:4]]), want_other, dtype)
    close(torch.cat([first[7:], second[:3]]), want[:8], dtype)


def attention_spec(hidden, nh, nkv, hd, theta, rotary, eps, window=None, qk_norm=True):
    from flyweight_amd.config import PartSpec
    return PartSpec("gqa_attention", {
        "hidden_size": hidden, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd, "qk_norm": qk_norm, "qk_norm_eps": eps,
        "window": window, "softmax_scale": 1 / math.sqrt(hd),
        "position": PartSpec("rotary_neox", {"theta": theta, "rotary_dim": rotary, "head_dim": hd}),
        "names": {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "out_proj", "q_norm": "q_layernorm", "k_norm": "k_layernorm"},
    }, prefix="a.")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,nh,nkv,hd,theta,eps", [(96, 6, 2, 16, 100.0, 1e-5), (144, 3, 3, 48, 1e6, 1e-6)])
def test_attention_part_whole_cut_and_batched(dtype, hidden, nh, nkv, hd, theta, eps):
    from flyweight_amd.parts import build_part
    part = build_part("mixer", attention_spec(hidden, nh, nkv, hd, theta, hd, eps))
    w = bound(part, dtype, seed=6)
    T = 150
    h = torch.randn(T, hidden, generator=torch.Generator().manual_seed(7)).to(dtype)
    config = {"num_attention_heads": nh, "num_key_value_heads": nkv, "hidden_size": nh * hd, "norm_eps": eps, "rope_theta": theta}
    want = plain.attention_mixer(h.double().numpy(), w, "a.", config)
    harness = Harness(part, dtype)
    close(harness.run([("whole", T)], h.to(DEV)), want, dtype)
    pieces, at = [], 0
    for n in (60, 4, 1, 1, 63, 2, 19):
        pieces.append(harness.run([("cut", n)], h[at:at + n].contiguous().to(DEV)))
        at += n
    close(torch.cat(pieces), want, dtype)
    # shifting every position changes nothing: only distances count (first 64 positions skipped)
    shifted = Harness(part, dtype)
    shifted.run([("s", 64)], torch.zeros(64, hidden, dtype=dtype, device=DEV))
    # ... but the zero rows are keys too, so compare with the plain model given the same prefix
    prefix = np.concatenate([np.zeros((64, hidden)), h[:40].double().numpy()])
    close(shifted.run([("s", 40)], h[:40].contiguous().to(DEV)), plain.attention_mixer(prefix, w, "a.", config)[64:], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_with_a_window_and_partial_rotation(dtype):
    """Options LFM2 does not use but the part takes as parameters."""
    from flyweight_amd.parts import build_part
    hidden, nh, nkv, hd, window, rotary = 64, 4, 2, 32, 70, 16
    part = build_part("mixer", attention_spec(hidden, nh, nkv, hd, 1e4, rotary, 1e-5, window=window, qk_norm=False))
    w = bound(part, dtype, seed=8)
    T = 200
    h = torch.randn(T, hidden, generator=torch.Generator().manual_seed(9)).to(dtype)
    x = h.double().numpy()
    q = (x @ w["a.q_proj.weight"].T).reshape(T, nh, hd)
    k = (x @ w["a.k_proj.weight"].T).reshape(T, nkv, hd)
    v = (x @ w["a.v_proj.weight"].T).reshape(T, nkv, hd)
    cos, sin = plain.rope_angles(np.arange(T), rotary, 1e4)
    q, k = plain.rope_half_split(q, cos, sin), plain.rope_half_split(k, cos, sin)
    want = plain.causal_attention(q, k, v, 1 / math.sqrt(hd), window=window).reshape(T, nh * hd) @ w["a.out_proj.weight"].T
    harness = Harness(part, dtype, num_pages=4)
    pieces, at = [], 0
    for n in (100, 1, 1, 30, 68):
        pieces.append(harness.run([("r", n)], h[at:at + n].contiguous().to(DEV)))
        at += n
    close(torch.cat(pieces), want, dtype)
    # the next query (position 200) sees keys 131..200: blocks 0 and 1 are passed, their pages back in the pool
    assert harness.cache.groups[0].tables["r"][:2] == [-1, -1] and harness.cache.groups[0].pool.in_use == 2


# ----- a toy mixer with state of its own ----------------------------------------------------
PRIOR_SUM, PRIOR_COUNT = 0.5, 2.0      # what the toy mixer's state starts with: not zero


def register_toy():
    from flyweight_amd.cache import CacheNeed
    from flyweight_amd.parts import Linear, Mixer, register_mixer
    from flyweight_amd.weights import TensorDecl

    class RunningSums(CacheNeed):
        """A need class of the toy's own: per request a running sum and a count, which start as if
        two tokens had been seen already. The cache manager stores it, hands out its slots and
        starts them by asking this class alone."""
        paged = False

        def __init__(self, width):
            self.width = width

        def __eq__(self, other):
            return isinstance(other, RunningSums) and other.width == self.width

        def __hash__(self):
            return hash(("running_sums", self.width))

        def allocate(self, units, page_size, dtype, device):
            return {"sums": torch.full((units, self.width), float("nan"), device=device),
                    "counts": torch.full((units,), float("nan"), device=device)}

        def initial(self, storage, slot):
            storage["sums"][slot] = PRIOR_SUM
            storage["counts"][slot] = PRIOR_COUNT

        def view(self, storage, block_table, writes):
            return storage

    @register_mixer("toy_running_mean")
    class RunningMean(Mixer):
        """out_t = W . (prior + h_0 + .. + h_t) / (prior count + t + 1)."""

        def __init__(self, spec):
            super().__init__(spec)
            self.hidden = int(spec["hidden_size"])

        def cache_need(self):
            return RunningSums(self.hidden)

        def tensors(self):
            return {self.prefix + "mix.weight": TensorDecl((self.hidden, self.hidden))}

        def bind(self, tensors, dtype, device):
            super().bind(tensors, dtype, device)
            self.mix = Linear(tensors[self.prefix + "mix.weight"])

        def forward(self, h, residual, ctx, cache):
            means = torch.empty_like(h)
            for seg in range(ctx.num_segments):
                lo, hi, slot = ctx.host_seg_row0[seg], ctx.host_seg_row0[seg + 1], ctx.host_seg_slot[seg]
                sums = cache["sums"][slot] + torch.cumsum(h[lo:hi].float(), dim=0)
                counts = cache["counts"][slot] + torch.arange(1, hi - lo + 1, device=h.device, dtype=torch.float32)
                means[lo:hi] = (sums / counts[:, None]).to(h.dtype)
                cache["sums"][slot] = sums[-1]
                cache["counts"][slot] = counts[-1]
            self.mix.accumulate(means, residual)
    return RunningMean


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_with_its_own_state_is_registered_built_and_stepped(tmp_path, dtype):
    from flyweight_amd.config import LayerSpec, PartSpec, ScheduleEntry, config_from_dict
    from flyweight_amd.engine import CausalLM, StepEntry, Stepper
    from flyweight_amd.engine.model import parse_dtype
    from flyweight_amd.weights import load_tensors, random_tensors, write_file
    from helpers import TINY_A
    register_toy()
    base = config_from_dict(TINY_A).model_spec()
    toy_layer = dataclasses.replace(base.layers[0], mixer=PartSpec("toy_running_mean", {"hidden_size": 64}, prefix="model.layers.0.toy."))
    # layers: toy, attention, conv, attention; the schedule runs the toy layer twice (two states)
    # and lets a second execution of layer 1 read the keys its first execution wrote
    spec = dataclasses.replace(base, layers=(toy_layer,) + base.layers[1:], schedule=(
        ScheduleEntry(0, cache=0), ScheduleEntry(1, cache=1), ScheduleEntry(2, cache=2), ScheduleEntry(0, cache=5),
        ScheduleEntry(1, cache=1, writes_cache=False), ScheduleEntry(3, cache=3)))
    model = CausalLM(spec)
    folder = str(tmp_path / "toy")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"), random_tensors(model.tensors(), 4, scale="fan_in"))
    torch_dtype = parse_dtype(dtype)
    tensors = load_tensors(folder, model.tensors(), torch_dtype, DEV)
    model.bind(tensors, torch_dtype, DEV)
    assert set(model.cache_needs()) == {0, 1, 2, 3, 5}
    w = {n: t.double().cpu().numpy() for n, t in tensors.items()}

    def expected(tokens):
        config = dict(TINY_A)
        eps = config["norm_eps"]
        x = w["model.embed_tokens.weight"][tokens]
        def toy(x):
            h = plain.rms_norm(x, w["model.layers.0.operator_norm.weight"], eps)
            means = (PRIOR_SUM + np.cumsum(h, axis=0)) / (PRIOR_COUNT + np.arange(1, len(h) + 1))[:, None]
            x = x + means @ w["model.layers.0.toy.mix.weight"].T
            return x + plain.swiglu(plain.rms_norm(x, w["model.layers.0.ffn_norm.weight"], eps), w, "model.layers.0.feed_forward.")
        def attention(x, i, reuse=None):
            p = f"model.layers.{i}."
            h = plain.rms_norm(x, w[p + "operator_norm.weight"], eps)
            T, nh, nkv, hd = len(x), 4, 2, 16
            q = plain.rms_norm((h @ w[p + "self_attn.q_proj.weight"].T).reshape(T, nh, hd), w[p + "self_attn.q_layernorm.weight"], eps)
            cos, sin = plain.rope_angles(np.arange(T), hd, config["rope_theta"])
            q = plain.rope_half_split(q, cos, sin)
            if reuse is None:
                k = plain.rms_norm((h @ w[p + "self_attn.k_proj.weight"].T).reshape(T, nkv, hd), w[p + "self_attn.k_layernorm.weight"], eps)
                reuse = (plain.rope_half_split(k, cos, sin), (h @ w[p + "self_attn.v_proj.weight"].T).reshape(T, nkv, hd))
            out = plain.causal_attention(q, reuse[0], reuse[1], 0.25).reshape(T, nh * hd) @ w[p + "self_attn.out_proj.weight"].T
            x = x + out
            return x + plain.swiglu(plain.rms_norm(x, w[p + "ffn_norm.weight"], eps), w, p + "feed_forward."), reuse
        def conv(x, i):
            p = f"model.layers.{i}."
            x = x + plain.short_conv_mixer(plain.rms_norm(x, w[p + "operator_norm.weight"], eps), w, p + "conv.", config)
            return x + plain.swiglu(plain.rms_norm(x, w[p + "ffn_norm.weight"], eps), w, p + "feed_forward.")
        x = toy(x)
        x, kv = attention(x, 1)
        x = conv(x, 2)
        x = toy(x)
        x, _ = attention(x, 1, reuse=kv)
        x, _ = attention(x, 3)
        return plain.rms_norm(x, w["model.embedding_norm.weight"], eps) @ w["model.embed_tokens.weight"].T

    rng = np.random.default_rng(0)
    a, b = rng.integers(0, 256, 90).tolist(), rng.integers(0, 256, 70).tolist()
    stepper = Stepper(model, num_pages=4, max_requests=2)
    stepper.admit("a"); stepper.admit("b")
    got = {"a": [], "b": []}
    plan = [[("a", 40)], [("a", 1), ("b", 30)], [("b", 2), ("a", 9)], [("a", 40), ("b", 38)]]
    at = {"a": 0, "b": 0}
    for step in plan:
        entries = []
        for request, n in step:
            tokens = (a if request == "a" else b)[at[request]:at[request] + n]
            entries.append(StepEntry(request, tokens, list(range(n))))
            at[request] += n
        logits = stepper.step(entries).cpu().numpy()
        row = 0
        for request, n in step:
            got[request].append(logits[row:row + n])
            row += n
    tolerance = {"float32": 2e-5, "bfloat16": 2e-2}[dtype]
    for request, tokens in (("a", a), ("b", b)):
        want = expected(tokens)
        found = np.concatenate(got[request])
        assert np.abs(found - want).max() <= tolerance * np.abs(want).max()
    # the toy state's slot is put back to its start for the next request
    stepper.release("a")
    stepper.admit("c")
    again = stepper.step([StepEntry("c", a[:20], list(range(20)))]).cpu().numpy()
    assert np.abs(again - expected(a[:20])).max() <= tolerance * np.abs(expected(a[:20])).max()


def register_toy_gate():
    from flyweight_amd.parts import Linear, Mixer, register_mixer
    from flyweight_amd.weights import TensorDecl

    @register_mixer("toy_position_gate")
    class PositionGate(Mixer):
        """out_t = W . (h_t * (1 + position_t mod 5)): the factor is built on the host from the rows'
        positions, an index array of the part's own that travels with every step's upload. The
        part launches device work only, so decode steps of a model that holds it are recorded;
        before each replay it brings its array up to date."""
        graph_safe = True
        refreshed = 0

        def __init__(self, spec):
            super().__init__(spec)
            self.hidden = int(spec["hidden_size"])

        def tensors(self):
            return {self.prefix + "mix.weight": TensorDecl((self.hidden, self.hidden))}

        def bind(self, tensors, dtype, device):
            super().bind(tensors, dtype, device)
            self.mix = Linear(tensors[self.prefix + "mix.weight"])

        def step_arrays_key(self):
            return ("toy_position_gate",)

        def step_arrays(self, batch):
            return {"gate": 1 + np.asarray(batch.host_row_pos, dtype=np.int32) % 5}

        def refresh_step_arrays(self, batch, arrays):
            arrays["gate"][:] = 1 + np.asarray(batch.host_row_pos, dtype=np.int32) % 5
            type(self).refreshed += 1

        def forward(self, h, residual, ctx, cache):
            gate = ctx.step_arrays(self)["gate"]
            self.mix.accumulate((h.float() * gate[:, None].float()).to(h.dtype), residual)
    return PositionGate


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_whose_index_array_depends_on_positions_is_replayed_from_recorded_steps(tmp_path, dtype):
    """A part's own index arrays may depend on the rows' positions and still ride in recorded
    decode steps: the step asks the part to refresh them before every replay. The logits are
    those of the plain computation, and bit for bit those of the same steps launched one by one."""
    from flyweight_amd.config import PartSpec, ScheduleEntry, config_from_dict
    from flyweight_amd.engine import CausalLM, StepEntry, Stepper
    from flyweight_amd.engine.model import parse_dtype
    from flyweight_amd.weights import load_tensors, random_tensors, write_file
    from helpers import TINY_A
    gate_class = register_toy_gate()
    base = config_from_dict(TINY_A).model_spec()
    toy_layer = dataclasses.replace(base.layers[0], mixer=PartSpec("toy_position_gate", {"hidden_size": 64}, prefix="model.layers.0.toy."))
    spec = dataclasses.replace(base, layers=(toy_layer,) + base.layers[1:], schedule=(
        ScheduleEntry(0, cache=None), ScheduleEntry(1, cache=1), ScheduleEntry(2, cache=2), ScheduleEntry(3, cache=3)))
    model = CausalLM(spec)
    folder = str(tmp_path / "gate")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"), random_tensors(model.tensors(), 6, scale="fan_in"))
    torch_dtype = parse_dtype(dtype)
    tensors = load_tensors(folder, model.tensors(), torch_dtype, DEV)
    model.bind(tensors, torch_dtype, DEV)
    w = {n: t.double().cpu().numpy() for n, t in tensors.items()}
    config = dict(TINY_A)
    eps = config["norm_eps"]

    def expected(tokens):
        x = w["model.embed_tokens.weight"][tokens]
        h = plain.rms_norm(x, w["model.layers.0.operator_norm.weight"], eps)
        x = x + (h * (1 + np.arange(len(tokens)) % 5)[:, None]) @ w["model.layers.0.toy.mix.weight"].T
        x = x + plain.swiglu(plain.rms_norm(x, w["model.layers.0.ffn_norm.weight"], eps), w, "model.layers.0.feed_forward.")
        for index, is_attention in ((1, True), (2, False), (3, True)):
            p = f"model.layers.{index}."
            h = plain.rms_norm(x, w[p + "operator_norm.weight"], eps)
            x = x + (plain.attention_mixer(h, w, p + "self_attn.", config) if is_attention else plain.short_conv_mixer(h, w, p + "conv.", config))
            x = x + plain.swiglu(plain.rms_norm(x, w[p + "ffn_norm.weight"], eps), w, p + "feed_forward.")
        return plain.rms_norm(x, w["model.embedding_norm.weight"], eps) @ w["model.embed_tokens.weight"].T

    rng = np.random.default_rng(3)
    a, b = rng.integers(0, 256, 40).tolist(), rng.integers(0, 256, 33).tolist()

    def run(recorded: bool):
        stepper = Stepper(model, num_pages=4, max_requests=2)
        assert stepper.use_graphs           # every part of the model, the toy too, allows recording
        stepper.use_graphs = recorded
        stepper.admit("a"); stepper.admit("b")
        got = {"a": [stepper.step([StepEntry("a", a[:20], list(range(20)))]).cpu().numpy()],
               "b": [stepper.step([StepEntry("b", b[:13], list(range(13)))]).cpu().numpy()]}
        for i in range(20):         # twenty decode steps of both requests, whose positions differ by seven
            out = stepper.step([StepEntry("a", a[20 + i:21 + i], [0]), StepEntry("b", b[13 + i:14 + i], [0])]).cpu().numpy()
            got["a"].append(out[:1]); got["b"].append(out[1:])
        return stepper, {name: np.concatenate(rows) for name, rows in got.items()}

    before = gate_class.refreshed
    stepper, recorded = run(True)
    assert stepper.graph_replays >= 18 and gate_class.refreshed - before == 20
    _, launched = run(False)
    tolerance = {"float32": 2e-5, "bfloat16": 3e-2}[dtype]
    for name, tokens in (("a", a), ("b", b)):
        want = expected(tokens)
        assert np.abs(recorded[name] - want).max() <= tolerance * np.abs(want).max()
        assert np.array_equal(recorded[name], launched[name])


# ----- a toy feed-forward with routing and a toy position encoding -----------------------------
TOY_STRETCH = 4.0
TOY_ROUTER_GAIN = 8.0       # router logits far apart: few rows sit near the border between the experts
TOY_TOKENS_SEED = 11      # with these tokens no row comes closer than 0.67
TOY_AMBIGUOUS = 0.5         # below this difference of router logits rounding may send a row the other way


def register_toy_router_and_positions():
    from flyweight_amd.kernels import ops
    from flyweight_amd.parts import FeedForward, Linear, register_feed_forward
    from flyweight_amd.parts.base import PositionEncoding, register_position_encoding
    from flyweight_amd.weights import TensorDecl

    @register_feed_forward("toy_top1_of_two")
    class TopOneOfTwo(FeedForward):
        """Two SwiGLU experts and a router: a row goes to the expert with the larger router logit
        (float32; ties to the first) and its output is weighted by the softmax share of that logit."""

        def __init__(self, spec):
            super().__init__(spec)
            self.hidden, self.width = int(spec["hidden_size"]), int(spec["intermediate_size"])

        def tensors(self):
            declared = {self.prefix + "router.weight": TensorDecl((2, self.hidden), "vector", "matrix")}
            for e in range(2):
                declared[f"{self.prefix}experts.{e}.gate_up.weight"] = TensorDecl((2 * self.width, self.hidden))
                declared[f"{self.prefix}experts.{e}.down.weight"] = TensorDecl((self.hidden, self.width))
            return declared

        def bind(self, tensors, dtype, device):
            super().bind(tensors, dtype, device)
            self.router = tensors[self.prefix + "router.weight"].float()
            self.experts = [(Linear(tensors[f"{self.prefix}experts.{e}.gate_up.weight"]),
                             Linear(tensors[f"{self.prefix}experts.{e}.down.weight"])) for e in range(2)]

        def forward(self, h, residual, ctx):
            logits = TOY_ROUTER_GAIN * (h.float() @ self.router.T)
            share = torch.softmax(logits, dim=-1)
            chosen = (logits[:, 1] > logits[:, 0]).long()
            for e, (gate_up, down) in enumerate(self.experts):
                rows = torch.nonzero(chosen == e).flatten()
                if rows.numel() == 0:
                    continue
                out = torch.zeros((rows.numel(), self.hidden), dtype=torch.float32, device=h.device)
                down.accumulate(gate_up.swiglu(h[rows].contiguous()), out)
                residual.index_add_(0, rows, out * share[rows, e, None])

    @register_position_encoding("toy_stretched_rotary")
    class StretchedRotary(PositionEncoding):
        """Half-split rotation by the angle of position / stretch: the tables the attention part's
        kernels take, made another way."""
        graph_safe = True

        def __init__(self, spec):
            super().__init__(spec)
            self.theta, self.rotary_dim, self.stretch = float(spec["theta"]), int(spec["head_dim"]), float(spec["stretch"])

        def bind(self, tensors, dtype, device):
            super().bind(tensors, dtype, device)
            half = self.rotary_dim // 2
            self.inv_freq = (self.theta ** (-(torch.arange(half, dtype=torch.float64) * 2.0 / self.rotary_dim)) / self.stretch).to(device)

        def tables(self, ctx):
            return ops.rope_table(ctx.encoding_pos, self.inv_freq)


def toy_spec(base):
    """Tiny A with a routed feed-forward and a stretched rotation in layer 1, scaled embeddings and
    scaled, capped logits."""
    from flyweight_amd.config import PartSpec
    layer = base.layers[1]
    position = PartSpec("toy_stretched_rotary", {"theta": 10000.0, "head_dim": 16, "stretch": TOY_STRETCH})
    mixer = dataclasses.replace(layer.mixer, params={**layer.mixer.params, "position": position})
    ffn = PartSpec("toy_top1_of_two", {"hidden_size": 64, "intermediate_size": 48}, prefix="model.layers.1.moe.")
    return dataclasses.replace(base, layers=(base.layers[0], dataclasses.replace(layer, mixer=mixer, ffn=ffn)) + base.layers[2:],
                               architecture="ToyForCausalLM", embedding_scale=1.5, logit_scale=0.5, logit_softcap=2.0)


def toy_expected_logits(w, tokens, shift=0):
    """Plain evaluation of ``toy_spec``'s model: (logits, first row whose routing is a close call)."""
    from helpers import TINY_A
    config = dict(TINY_A)
    eps = config["norm_eps"]
    x = 1.5 * w["model.embed_tokens.weight"][tokens]
    T = len(tokens)
    close_call = T
    for i, is_attention in enumerate(plain.attention_layers(config)):
        p = f"model.layers.{i}."
        h = plain.rms_norm(x, w[p + "operator_norm.weight"], eps)
        if is_attention:
            positions = (np.arange(T) + shift) / (TOY_STRETCH if i == 1 else 1.0)
            q, k, v = plain.attention_qkv(h, w, p + "self_attn.", config, positions)
            x = x + plain.causal_attention(q, k, v, 0.25).reshape(T, -1) @ w[p + "self_attn.out_proj.weight"].T
        else:
            x = x + plain.short_conv_mixer(h, w, p + "conv.", config)
        h = plain.rms_norm(x, w[p + "ffn_norm.weight"], eps)
        if i == 1:
            logits = TOY_ROUTER_GAIN * (h @ w[p + "moe.router.weight"].T)
            share = np.exp(logits - logits.max(-1, keepdims=True))
            share /= share.sum(-1, keepdims=True)
            near = np.nonzero(np.abs(logits[:, 1] - logits[:, 0]) < TOY_AMBIGUOUS)[0]
            close_call = int(near[0]) if len(near) else T
            x = x.copy()
            for t in range(T):
                e = int(logits[t, 1] > logits[t, 0])
                both = h[t] @ w[f"{p}moe.experts.{e}.gate_up.weight"].T
                x[t] = x[t] + share[t, e] * ((plain.silu(both[:48]) * both[48:]) @ w[f"{p}moe.experts.{e}.down.weight"].T)
        else:
            x = x + plain.swiglu(h, w, p + "feed_forward.")
    logits = 0.5 * (plain.rms_norm(x, w["model.embedding_norm.weight"], eps) @ w["model.embed_tokens.weight"].T)
    return 2.0 * np.tanh(logits / 2.0), close_call


def test_a_toy_architecture_is_registered_and_served_from_a_folder(tmp_path):
    """An architecture of this file's own (its configuration class, its key names, its parts) goes
    through the registry: a model folder is written from its configuration and a seed, opened by
    name as any folder is, and generates through the runtime (scheduler, prompt portions, decode
    steps) the tokens of a plain evaluation. Nothing of the package knows it."""
    import flyweight_amd
    from flyweight_amd.config import config_from_dict, register_architecture, registered_architectures
    from flyweight_amd.weights import write_random_model
    from helpers import TINY_A
    register_toy_router_and_positions()

    class ToyConfig:
        """config.json of the toy: {"architectures": ["ToyForCausalLM"], "base": <an LFM2 config>}."""

        def __init__(self, base):
            self.base = base

        @classmethod
        def from_dict(cls, data):
            return cls(config_from_dict(data["base"]))

        def model_spec(self):
            return toy_spec(self.base.model_spec())

        def save(self, folder):
            import json
            with open(os.path.join(folder, "config.json"), "w") as handle:
                json.dump({"architectures": ["ToyForCausalLM"], "base": self.base.to_dict()}, handle)

    register_architecture("ToyForCausalLM", ToyConfig, replace=True)
    assert "ToyForCausalLM" in registered_architectures()
    folder = write_random_model(str(tmp_path / "toy3"), ToyConfig(config_from_dict(TINY_A)), seed=9, scale="fan_in")
    model = flyweight_amd.Model(folder, dtype="float32")
    assert isinstance(model.config, ToyConfig) and model.spec.architecture == "ToyForCausalLM"
    from safetensors.torch import load_file
    w = {n: t.double().numpy() for n, t in load_file(os.path.join(folder, "model.safetensors")).items()}
    prompt = np.random.default_rng(TOY_TOKENS_SEED).integers(0, 256, 45).tolist()
    expected, tokens = [], list(prompt)
    for _ in range(6):
        logits, _ = toy_expected_logits(w, tokens)
        expected.append(plain.most_likely(logits[-1]))
        tokens.append(expected[-1])
    with flyweight_amd.Runtime(model, parallel_sequences=2, prefill_rows=16, max_batch_tokens=24) as runtime:
        other = runtime.task_submit(prompt[:20], 3)         # a second request beside it: mixed steps
        assert runtime.generate(prompt, 6) == expected
        runtime.run()
        assert runtime.task_error(other) is None and runtime.info["live_requests"] == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routing_feed_forward_and_position_encoding_need_no_change_to_the_framework(tmp_path, dtype):
    """Layer 1 of tiny A gets a routed feed-forward and a stretched rotation, both defined in this
    file; the model also scales its embeddings and caps its logits (``ModelSpec`` fields no LFM2
    uses). Whole prompt against portions and decoded tokens, against a plain evaluation; and a
    shift of the positions that the encoding sees leaves the logits where they were."""
    from flyweight_amd.config import PartSpec, config_from_dict
    from flyweight_amd.engine import CausalLM, StepEntry, Stepper
    from flyweight_amd.engine.model import parse_dtype
    from flyweight_amd.weights import load_tensors, random_tensors, write_file
    from helpers import TINY_A
    register_toy_router_and_positions()
    spec = toy_spec(config_from_dict(TINY_A).model_spec())
    model = CausalLM(spec)
    folder = str(tmp_path / "toy2")
    os.makedirs(folder)
    write_file(os.path.join(folder, "model.safetensors"), random_tensors(model.tensors(), 9, scale="fan_in"))
    torch_dtype = parse_dtype(dtype)
    tensors = load_tensors(folder, model.tensors(), torch_dtype, DEV)
    model.bind(tensors, torch_dtype, DEV)
    w = {n: t.double().cpu().numpy() for n, t in tensors.items()}
    config = dict(TINY_A)
    eps = config["norm_eps"]

    def expected(tokens, shift=0):
        return toy_expected_logits(w, tokens, shift)

    tokens = np.random.default_rng(TOY_TOKENS_SEED).integers(0, 256, 100).tolist()
    want, sure = expected(tokens)
    assert sure >= 60                                           # chosen so: most rows are compared in bfloat16 too
    compared = 100 if dtype == "float32" else sure
    assert 0.3 < np.abs(want).max() < 2.0                      # the cap bends the logits but does not flatten them
    stepper = Stepper(model, num_pages=6, max_requests=3)
    tolerance = {"float32": 2e-5, "bfloat16": 3e-2}[dtype]
    for request, cuts in (("whole", [100]), ("cut", [7, 2, 30, 1, 1, 1, 58])):
        stepper.admit(request)
        found, at = [], 0
        for n in cuts:
            found.append(stepper.step([StepEntry(request, tokens[at:at + n], list(range(n)))]).cpu().numpy())
            at += n
        assert np.abs(np.concatenate(found) - want)[:compared].max() <= tolerance * np.abs(want).max(), request
    # positions are the encoding's business: shifted by a constant, only distances count, and the
    # cache and the mask still follow the order of the tokens
    stepper.admit("shifted")
    found, at = [], 0
    for n in (40, 1, 59):
        entry = StepEntry("shifted", tokens[at:at + n], list(range(n)), positions=list(range(1000 + at, 1000 + at + n)))
        found.append(stepper.step([entry]).cpu().numpy())
        at += n
    shifted = np.concatenate(found)
    want_shifted, sure_shifted = expected(tokens, shift=1000)
    compared = 100 if dtype == "float32" else min(sure, sure_shifted)
    assert np.abs(shifted - want_shifted)[:compared].max() <= tolerance * np.abs(want).max()
    assert np.abs(shifted - want)[:compared].max() <= 2 * tolerance * np.abs(want).max()
    with pytest.raises(Exception, match="positions"):
        stepper.step([StepEntry("shifted", [1, 2], [], positions=[5])])
