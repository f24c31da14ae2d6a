"""Each part alone against the plain implementation, and parts of other kinds, defined here,
registered, built and stepped without a change to the framework's files."""

from dataclasses import dataclass
from types import SimpleNamespace
from typing import Optional

import pytest
import torch

from tests import helpers
from tests.plain import moondream_plain as plain

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]
IDS = ["fp32", "bf16"]


def _tensors(part, dtype, seed, std=0.2):
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in part.params().items():
        noise = torch.randn(spec.shape, generator=gen)
        value = 1 + 0.1 * noise if spec.init == "gain" else std * noise
        out[name] = value.to(torch.bfloat16).to(dtype if spec.role == "matrix" else torch.float32)
    return out


def _workspace_batch(n_tokens, **extra):
    from kestrel_amd.engine.batch import Workspace

    return SimpleNamespace(workspace=Workspace(DEV), n_tokens=n_tokens, **extra)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_layernorm_part(dtype):
    from kestrel_amd.parts import NormSpec, build_part

    part = build_part("norm", NormSpec("layernorm", 200, 3e-4, bias=True))
    weights = _tensors(part, dtype, 0)
    part.bind(weights, dtype, DEV)
    x = torch.randn(7, 200) * 2 + 0.5
    out = torch.empty(7, 200, dtype=dtype, device=DEV)
    part.forward(x.to(DEV), out)
    ref = plain.layer_norm(x.double(), weights["weight"].double(), weights["bias"].double(), 3e-4)
    helpers.assert_close(out, ref, dtype, "layernorm part")


def test_rotary_table_part():
    from kestrel_amd.parts import PositionSpec, build_part

    part = build_part("position", PositionSpec("rotary_neox", 12, 1234.5, 77))
    table = part.table(DEV)
    assert table.dtype == torch.float32 and tuple(table.shape) == (77, 12)
    torch.testing.assert_close(table.cpu().double(), plain.rotary_table(12, 77, 1234.5), atol=2e-5, rtol=0)
    assert build_part("position", PositionSpec("none")).rotation(DEV) is None
    rotation = part.rotation(DEV)
    assert rotation.pairing == "halves" and rotation.table is table


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_feed_forward_part(dtype):
    from kestrel_amd.parts import DenseFeedForwardSpec, build_part

    part = build_part("feed_forward", DenseFeedForwardSpec("dense", 72, 200, "gelu_tanh", bias=True))
    w = _tensors(part, dtype, 1)
    part.bind(w, dtype, DEV)
    h = (torch.randn(9, 72)).to(torch.bfloat16)
    residual = torch.randn(9, 72)
    out = residual.clone().to(DEV)
    part.forward(h.to(dtype).to(DEV), _workspace_batch(9), out)
    wd = {"p.mlp." + k: v.double() for k, v in w.items()}
    ref = residual.double() + plain.mlp(h.double(), wd, "p.")
    helpers.assert_close(out, ref, dtype, "feed-forward part")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(4, 4, 16, 8), (6, 2, 48, 12), (3, 1, 64, 32)])
def test_attention_part(shape, dtype):
    """The mixer alone on a cache of its own: a prompt in two portions, then a decoded token."""
    from kestrel_amd.cache import CacheManager
    from kestrel_amd.engine.step import ModelRunner, StepEntry
    from kestrel_amd.parts import AttentionSpec, PositionSpec, build_part

    h, hkv, hd, rot = shape
    dim = 40
    spec = AttentionSpec("attention", dim, h, hkv, hd, PositionSpec("rotary_neox", rot, 500.0, 64), bias=True)
    part = build_part("mixer", spec)
    w = _tensors(part, dtype, 2, std=0.08)         # outputs of order 0.3: the tolerances are absolute
    part.bind(w, dtype, DEV)
    cache = CacheManager([(part.cache_spec(), None, None)], 16, 8, 2, dtype=dtype, device=DEV)
    fake_model = SimpleNamespace(plan=SimpleNamespace(max_positions=64, vocab_size=10, dim=dim))
    runner = ModelRunner(fake_model, cache, DEV)
    slot = runner.admit()
    total = 23
    hs = torch.randn(total, dim).to(torch.bfloat16)
    outs = []
    for lo, hi in ((0, 17), (17, 22), (22, 23)):
        batch = runner.build_batch([StepEntry(slot, [1] * (hi - lo))])
        residual = torch.zeros(hi - lo, dim, device=DEV)
        part.forward(hs[lo:hi].to(dtype).to(DEV), batch, runner.layer_caches[0], residual)
        runner.held[slot] = hi
        outs.append(residual.cpu())
    cfg = {"n_heads": h, "n_kv_heads": hkv, "head_dim": hd}
    wd = {"p.attn." + k: v.double() for k, v in w.items()}
    positions = torch.arange(total)
    ref = plain.attention(hs.double(), wd, "p.", cfg, positions, plain.visibility(positions, None),
                          plain.rotary_table(rot, 64, 500.0))
    helpers.assert_close(torch.cat(outs), ref, dtype, f"attention part {shape}")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(4, 2, 32, 16), (2, 2, 64, 64), (3, 1, 48, 20)])
def test_another_position_encoding_in_the_attention_mixer(shape, dtype):
    """A rotary encoding that pairs neighbouring channels (2i with 2i + 1), registered from here:
    the attention mixer takes its ``Rotation`` and the kernels turn the pairs it names. Turning
    neighbours equals turning halves after moving the even channels of the rotated part of every
    query and key head to the front, and scores do not change when queries and keys are permuted
    alike: the plain implementation with the rows of the q|k weights permuted that way is the
    reference. Also: an encoding that holds a table but offers no rotation is refused."""
    from kestrel_amd.cache import CacheManager
    from kestrel_amd.engine.step import ModelRunner, StepEntry
    from kestrel_amd.parts import AttentionSpec, PositionEncoding, PositionSpec, Rotation, build_part, register_position

    class PairsRotary(PositionEncoding):
        def rotation(self, device):
            spec = self.spec
            return Rotation(plain.rotary_table(spec.rotary_dim, spec.max_positions, spec.theta, torch.float32).to(device),
                            "interleaved")

    class TableOnly(PositionEncoding):
        def table(self, device):
            return torch.zeros(4, 8, device=device)

    register_position("toy_rotary_pairs", PairsRotary)
    register_position("toy_table_only", TableOnly)
    h, hkv, hd, rot = shape
    dim = 40
    spec = AttentionSpec("attention", dim, h, hkv, hd, PositionSpec("toy_rotary_pairs", rot, 300.0, 64), bias=True)
    part = build_part("mixer", spec)
    w = _tensors(part, dtype, 5, std=0.08)
    part.bind(w, dtype, DEV)
    cache = CacheManager([(part.cache_spec(), None, None)], 16, 8, 2, dtype=dtype, device=DEV)
    fake_model = SimpleNamespace(plan=SimpleNamespace(max_positions=64, vocab_size=10, dim=dim))
    runner = ModelRunner(fake_model, cache, DEV)
    slot = runner.admit()
    total = 39
    hs = torch.randn(total, dim, generator=torch.Generator().manual_seed(8)).to(torch.bfloat16)
    outs = []
    for lo, hi in ((0, 18), (18, 35), (35, 36), (36, 37), (37, 39)):
        batch = runner.build_batch([StepEntry(slot, [1] * (hi - lo))])
        residual = torch.zeros(hi - lo, dim, device=DEV)
        part.forward(hs[lo:hi].to(dtype).to(DEV), batch, runner.layer_caches[0], residual)
        runner.held[slot] = hi
        outs.append(residual.cpu())
    order = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, hd))     # evens of the rotated part first
    rows = [head * hd + c for head in range(h + hkv) for c in order] + list(range((h + hkv) * hd, (h + 2 * hkv) * hd))
    wd = {"p.attn." + k: v.double() for k, v in w.items()}
    wd["p.attn.qkv.weight"], wd["p.attn.qkv.bias"] = wd["p.attn.qkv.weight"][rows], wd["p.attn.qkv.bias"][rows]
    cfg = {"n_heads": h, "n_kv_heads": hkv, "head_dim": hd}
    positions = torch.arange(total)
    ref = plain.attention(hs.double(), wd, "p.", cfg, positions, plain.visibility(positions, None),
                          plain.rotary_table(rot, 64, 300.0))
    helpers.assert_close(torch.cat(outs), ref, dtype, f"attention with paired rotary {shape}")
    halves = plain.attention(hs.double(), {"p.attn." + k: v.double() for k, v in w.items()}, "p.", cfg, positions,
                             plain.visibility(positions, None), plain.rotary_table(rot, 64, 300.0))
    assert (halves - ref).abs().max() > 0.02, "the two pairings must differ on this input, or the test shows nothing"
    with pytest.raises(ValueError, match="offers no rotation"):
        bad = build_part("mixer", AttentionSpec("attention", dim, h, hkv, hd, PositionSpec("toy_table_only", rot, 300.0, 64)))
        bad.bind(_tensors(bad, dtype, 5), dtype, DEV)


# ------------------------------------------------------------------------------------------------
# parts of other kinds, defined in this test file
# ------------------------------------------------------------------------------------------------

@dataclass(frozen=True)
class DecaySpec:
    kind: str
    dim: int
    decay: float


def _register_toys():
    from kestrel_amd.parts import (FeedForward, Mixer, ParamSpec, PositionEncoding, StateSpec, register_feed_forward,
                                   register_mixer, register_position)

    class DecayMixer(Mixer):
        """A mixer with state of its own and no keys or values: ``s <- decay * s + h W``, output ``s``.
        The state lives in the cache manager's per-request slots."""

        def params(self):
            return {"w.weight": ParamSpec((self.spec.dim, self.spec.dim))}

        def state_spec(self):
            return StateSpec((self.spec.dim,), "float32")

        def bind(self, tensors, dtype, device):
            self.w = tensors["w.weight"].to(device).float()

        def forward(self, h, batch, cache, residual):
            # torch and the framework's plain linear on the GPU: this toy shows the interfaces, not a kernel
            from kestrel_amd.ops.linear import linear

            u = batch.workspace.get("toy.u", tuple(h.shape), torch.float32)
            linear(h.float(), self.w, None, u)
            if batch.decode_only:
                # one token per row, nothing here looks at values on the host: this can be captured
                # in a graph. Rows that pad the batch have slot -1, the state's spare last row.
                slots = batch.row_slot.long()[batch.token_row.long()]
                state = self.spec.decay * cache.state[slots] + u
                cache.state[slots] = state
                residual += state
                return
            rows = batch.token_row.long()
            slots = batch.row_slot.long()
            for t in range(h.shape[0]):
                slot = slots[rows[t]]
                if slot < 0:
                    continue
                cache.state[slot] = self.spec.decay * cache.state[slot] + u[t]
                residual[t] += cache.state[slot]

    class RoutedFeedForward(FeedForward):
        """A feed-forward with routing: the router picks one of two experts per token."""

        def params(self):
            d = self.spec.dim
            return {"router.weight": ParamSpec((2, d)), "e0.weight": ParamSpec((d, d)), "e1.weight": ParamSpec((d, d))}

        def bind(self, tensors, dtype, device):
            self.t = {k: v.to(device).float() for k, v in tensors.items()}

        def forward(self, h, batch, residual):
            from kestrel_amd.ops.linear import linear

            x = h.float()
            n, d = x.shape
            scores = batch.workspace.get("toy.router", (n, 2), torch.float32)     # fixed addresses: safe in a graph
            both = batch.workspace.get("toy.experts", (2, n, d), torch.float32)
            linear(x, self.t["router.weight"], None, scores)
            linear(x, self.t["e0.weight"], None, both[0])
            linear(x, self.t["e1.weight"], None, both[1])
            second = (scores[:, 1] > scores[:, 0]).unsqueeze(1)                    # argmax of two, first wins a tie
            residual += torch.where(second, both[1], both[0])

    class LearnedPosition(PositionEncoding):
        """Another position encoding: nothing to rotate, so no table."""

    register_mixer("toy_decay", DecayMixer)
    register_feed_forward("toy_routed", RoutedFeedForward)
    register_position("toy_learned", LearnedPosition)


def _toy_reference(ids, w, decay, eps):
    """The toy model computed plainly: layer 0 (decay mixer, routed ff, sequential norms), then
    layer 1 = attention + dense, then layer 0 again (its weights, a state of its own)."""
    dim = w["emb"].shape[1]
    x = w["emb"].double()[torch.tensor(ids)]
    positions = torch.arange(len(ids))
    allowed = plain.visibility(positions, None)

    def toy_layer(x, state):
        out = []
        for t in range(x.shape[0]):
            xt = x[t]
            h = plain.layer_norm(xt, w["l0.n1.weight"].double(), w["l0.n1.bias"].double(), eps)
            state = decay * state + w["l0.mix.w.weight"].double() @ h
            xt = xt + state
            h2 = plain.layer_norm(xt, w["l0.n2.weight"].double(), w["l0.n2.bias"].double(), eps)
            e = int((w["l0.ff.router.weight"].double() @ h2).argmax())
            xt = xt + w[f"l0.ff.e{e}.weight"].double() @ h2
            out.append(xt)
        return torch.stack(out)

    x = toy_layer(x, torch.zeros(dim, dtype=torch.float64))
    cfg = {"n_heads": 2, "n_kv_heads": 1, "head_dim": 16}
    wd = {k.replace("l1.", "p."): v.double() for k, v in w.items() if k.startswith("l1.")}
    xn = plain.layer_norm(x, wd["p.ln.weight"], wd["p.ln.bias"], eps)
    x = x + plain.attention(xn, wd, "p.", cfg, positions, allowed, plain.rotary_table(8, 64, 100.0)) \
        + plain.mlp(xn, wd, "p.")
    x = toy_layer(x, torch.zeros(dim, dtype=torch.float64))
    normed = plain.layer_norm(x, w["fn.weight"].double(), w["fn.bias"].double(), eps)
    return normed @ w["emb"].double().T          # tied head, no bias


def _toy_model():
    """The toy plan (a layer with a stateful mixer and a routed feed-forward, named twice around
    an attention layer), its bound model and its weights."""
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.parts import (AttentionSpec, DenseFeedForwardSpec, LayerSpec, ModelPlan, NormSpec, PositionSpec,
                                   ScheduleEntry)

    _register_toys()
    dim, vocab, eps, decay = 32, 50, 1e-5, 0.5
    norm = NormSpec("layernorm", dim, eps)
    toy = LayerSpec("sequential", norm, DecaySpec("toy_decay", dim, decay), DecaySpec("toy_routed", dim, 0.0),
                    norm2=norm, names={"norm.weight": "l0.n1.weight", "norm.bias": "l0.n1.bias",
                                       "norm2.weight": "l0.n2.weight", "norm2.bias": "l0.n2.bias",
                                       "mixer.w.weight": "l0.mix.w.weight",
                                       "feed_forward.router.weight": "l0.ff.router.weight",
                                       "feed_forward.e0.weight": "l0.ff.e0.weight",
                                       "feed_forward.e1.weight": "l0.ff.e1.weight"})
    attn = LayerSpec("parallel", norm,
                     AttentionSpec("attention", dim, 2, 1, 16, PositionSpec("rotary_neox", 8, 100.0, 64)),
                     DenseFeedForwardSpec("dense", dim, 48),
                     names={"norm.weight": "l1.ln.weight", "norm.bias": "l1.ln.bias",
                            "mixer.qkv.weight": "l1.attn.qkv.weight", "mixer.qkv.bias": "l1.attn.qkv.bias",
                            "mixer.proj.weight": "l1.attn.proj.weight", "mixer.proj.bias": "l1.attn.proj.bias",
                            "feed_forward.fc1.weight": "l1.mlp.fc1.weight", "feed_forward.fc1.bias": "l1.mlp.fc1.bias",
                            "feed_forward.fc2.weight": "l1.mlp.fc2.weight", "feed_forward.fc2.bias": "l1.mlp.fc2.bias"})
    plan = ModelPlan("toy", vocab, dim, 64, (toy, attn), (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)),
                     norm, head_bias=False, tied_head=True,
                     names={"embedding": "emb", "final_norm.weight": "fn.weight", "final_norm.bias": "fn.bias"})
    model = DecoderModel(plan)
    gen = torch.Generator().manual_seed(3)
    weights = {}
    for name, spec in model.params().items():
        noise = torch.randn(spec.shape, generator=gen)
        weights[name] = (1 + 0.1 * noise) if spec.init == "gain" else 0.3 * noise
    model.bind(weights, torch.float32, DEV)
    return model, weights, vocab, eps, decay


def test_a_stateful_toy_mixer_is_stepped_once_per_replayed_step():
    """The toy model with HIP graphs on: decode steps of two, then three live requests (buckets of
    2 and 4, the second with a padding row) are replayed. A graph is captured and warmed up on
    padding rows alone, so the state of a live request is advanced exactly once a step: every
    replay's logits match the plain computation, with eager prompt steps between the replays."""
    from kestrel_amd.cache import CacheManager
    from kestrel_amd.engine.step import ModelRunner, StepEntry

    model, weights, vocab, eps, decay = _toy_model()
    cache = CacheManager(model.cache_needs(), 16, 12, 4, dtype=torch.float32, device=DEV)
    runner = ModelRunner(model, cache, DEV, enable_graphs=True)
    seqs = {name: helpers.random_ids(60 + i, n, vocab) for i, (name, n) in enumerate((("a", 30), ("b", 24), ("c", 19)))}
    expected = {name: _toy_reference(ids, weights, decay, eps) for name, ids in seqs.items()}
    slots, fed = {}, {}

    def prompt(name, count):
        slots[name] = runner.admit()
        out = runner.step([StepEntry(slots[name], seqs[name][:count], want=[count - 1])]).clone()
        fed[name] = count
        helpers.assert_close(out[0], expected[name][count - 1], torch.float32, f"toy prompt {name}")

    def decode(names, what):
        entries = [StepEntry(slots[n], [seqs[n][fed[n]]], want=[0]) for n in names]
        before = runner.graph_replays
        out = runner.step(entries).clone()
        assert runner.graph_replays == before + 1
        for i, n in enumerate(names):
            helpers.assert_close(out[i], expected[n][fed[n]], torch.float32, f"{what}: request {n} at {fed[n]}")
            fed[n] += 1

    prompt("a", 9)
    prompt("b", 5)
    for i in range(4):                       # bucket 2: the first of these steps captures the graph
        decode(["a", "b"], f"bucket 2, replay {i}")
    prompt("c", 7)                           # eager work between replays
    for i in range(4):                       # bucket 4 with one padding row
        decode(["c", "a", "b"], f"bucket 4, replay {i}")
    runner.release(slots.pop("b"))
    for i in range(3):                       # back to the first graph, other rows
        decode(["a", "c"], f"bucket 2 again, replay {i}")
    prompt("b", 11)                          # the freed slot is used again and starts from a zero state
    for i in range(3):
        decode(["b", "c", "a"], f"bucket 4 again, replay {i}")
    assert sorted(runner._graphs) == [2, 4]
    # the toy parts do not promise to be replayable in steps of every shape: the prompts were launched kernel by kernel
    assert not runner.mixed_graphs and runner.mixed_graph_replays == 0 and not runner._mixed


def test_toy_parts_build_and_step():
    """A mixer with state, a routed feed-forward and another position encoding are registered
    from here; a plan names a layer twice in its schedule; the generic decoder, the cache
    manager and the step function run it in portions and match a plain computation."""
    from kestrel_amd.cache import CacheManager
    from kestrel_amd.engine.step import ModelRunner, StepEntry

    model, weights, vocab, eps, decay = _toy_model()
    needs = model.cache_needs()
    assert [n[0] is None for n in needs] == [True, False, True] and [n[1] is None for n in needs] == [False, True, False]
    cache = CacheManager(needs, 16, 8, 3, dtype=torch.float32, device=DEV)
    assert cache.states[0] is not None and cache.states[2] is not None and cache.states[0] is not cache.states[2]
    runner = ModelRunner(model, cache, DEV)
    ids_a = helpers.random_ids(30, 21, vocab)
    ids_b = helpers.random_ids(31, 9, vocab)
    a, b = runner.admit(), runner.admit()
    got_a, got_b = [], []
    out = runner.step([StepEntry(a, ids_a[:12], want=list(range(12)))]).clone()
    got_a.append(out)
    out = runner.step([StepEntry(a, ids_a[12:20], want=list(range(8))), StepEntry(b, ids_b[:8], want=list(range(8)))]).clone()
    got_a.append(out[:8])
    got_b.append(out[8:])
    out = runner.step([StepEntry(b, ids_b[8:], want=[0]), StepEntry(a, ids_a[20:], want=[0])]).clone()
    got_b.append(out[:1])
    got_a.append(out[1:])
    helpers.assert_close(torch.cat(got_a), _toy_reference(ids_a, weights, decay, eps), torch.float32, "toy a")
    helpers.assert_close(torch.cat(got_b), _toy_reference(ids_b, weights, decay, eps), torch.float32, "toy b")
    # a slot that is used again starts from a zero state
    runner.release(a)
    c = runner.admit()
    assert c == a
    out = runner.step([StepEntry(c, ids_b, want=list(range(9)))]).clone()
    helpers.assert_close(out, _toy_reference(ids_b, weights, decay, eps), torch.float32, "toy c")


@dataclass(frozen=True)
class LatentCacheSpec:
    """What the toy mixer below keeps per token: one vector, pages of ``[page_size, width]``."""

    width: int
    window: Optional[int] = None

    def page_tensors(self, page_size):
        return {"c": (page_size, self.width)}

    @property
    def group_key(self):
        return ("latent", self.width, self.window)


@dataclass(frozen=True)
class LatentSpec:
    kind: str
    dim: int
    width: int


def test_a_mixer_with_a_cache_layout_of_its_own():
    """A toy mixer that caches one latent per token (no keys, no values) in pages whose layout its
    own specification names: the cache manager allocates what the specification says, gives the
    layer its slice, and pages, block tables, slots and reuse work as for attention. The layer
    stands beside an attention layer, which gets a group and a pool of its own."""
    from kestrel_amd.cache import CacheManager
    from kestrel_amd.engine.step import ModelRunner
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.ops.linear import linear
    from kestrel_amd.parts import (AttentionSpec, DenseFeedForwardSpec, LayerSpec, Mixer, ModelPlan, NormSpec, ParamSpec,
                                   PositionSpec, ScheduleEntry, register_mixer)

    class LatentMixer(Mixer):
        """``c_t = h_t Wc`` is cached; the output at ``t`` is ``mean_{j <= t}(c_j) Wo``."""

        def params(self):
            return {"down.weight": ParamSpec((self.spec.width, self.spec.dim)), "up.weight": ParamSpec((self.spec.dim, self.spec.width))}

        def cache_spec(self):
            return LatentCacheSpec(self.spec.width)

        def bind(self, tensors, dtype, device):
            self.down, self.up = tensors["down.weight"].to(device).float(), tensors["up.weight"].to(device).float()

        def forward(self, h, batch, cache, residual):
            group = batch.groups[cache.group]
            store = cache.tensors["c"]                              # [pages, page_size, width]
            flat = store.view(-1, store.shape[-1])
            n = h.shape[0]
            latent = batch.workspace.get("toy.latent", (n, self.spec.width), torch.float32)
            linear(h.float(), self.down, None, latent)
            flat[group.slots.long()] = latent.to(flat.dtype)       # write before read, as attention does
            means = torch.zeros(n, self.spec.width, device=h.device)
            rows, hi = batch.token_row.tolist(), batch.kv_hi.tolist()
            for t in range(n):
                pages = group.block_table[rows[t], : -(-hi[t] // group.page_size)].long()
                means[t] = store[pages].reshape(-1, store.shape[-1])[:hi[t]].float().mean(dim=0)
            out = batch.workspace.get("toy.latent_out", (n, self.spec.dim), torch.float32)
            linear(means, self.up, None, out)
            residual += out

    register_mixer("toy_latent", LatentMixer)
    dim, vocab, eps, width = 32, 60, 1e-5, 12
    norm = NormSpec("layernorm", dim, eps)
    ff_names = {"feed_forward.fc1.weight": "{}.fc1.weight", "feed_forward.fc1.bias": "{}.fc1.bias",
                "feed_forward.fc2.weight": "{}.fc2.weight", "feed_forward.fc2.bias": "{}.fc2.bias",
                "norm.weight": "{}.ln.weight", "norm.bias": "{}.ln.bias"}
    toy = LayerSpec("parallel", norm, LatentSpec("toy_latent", dim, width), DenseFeedForwardSpec("dense", dim, 40),
                    names={**{k: v.format("l0") for k, v in ff_names.items()}, "mixer.down.weight": "l0.down", "mixer.up.weight": "l0.up"})
    attn = LayerSpec("parallel", norm, AttentionSpec("attention", dim, 2, 1, 16, PositionSpec("rotary_neox", 8, 100.0, 96)),
                     DenseFeedForwardSpec("dense", dim, 40),
                     names={**{k: v.format("l1") for k, v in ff_names.items()}, "mixer.qkv.weight": "l1.attn.qkv.weight",
                            "mixer.qkv.bias": "l1.attn.qkv.bias", "mixer.proj.weight": "l1.attn.proj.weight",
                            "mixer.proj.bias": "l1.attn.proj.bias"})
    plan = ModelPlan("toy-latent", vocab, dim, 96, (toy, attn), (ScheduleEntry(0), ScheduleEntry(1)), norm, head_bias=False,
                     tied_head=True, names={"embedding": "emb", "final_norm.weight": "fn.weight", "final_norm.bias": "fn.bias"})
    model = DecoderModel(plan)
    gen = torch.Generator().manual_seed(9)
    weights = {}
    for name, spec in model.params().items():
        noise = torch.randn(spec.shape, generator=gen)
        weights[name] = (1 + 0.1 * noise) if spec.init == "gain" else 0.3 * noise
    model.bind(weights, torch.float32, DEV)
    cache = CacheManager(model.cache_needs(), 16, 9, 3, dtype=torch.float32, device=DEV)
    assert len(cache.groups) == 2 and set(cache.groups[0].tensors) == {"c"} and set(cache.groups[1].tensors) == {"k", "v"}
    assert tuple(cache.groups[0].tensors["c"].shape) == (1, 9, 16, width)
    assert cache.bytes_per_page() == 4 * (16 * width + 2 * 16 * 16)
    runner = ModelRunner(model, cache, DEV)
    helpers.poison_cache(runner)

    def reference(ids):
        w = {k: v.double() for k, v in weights.items()}
        x = w["emb"][torch.tensor(ids)]
        positions = torch.arange(len(ids))
        h = plain.layer_norm(x, w["l0.ln.weight"], w["l0.ln.bias"], eps)
        latent = h @ w["l0.down"].T
        means = torch.cumsum(latent, dim=0) / (positions + 1).unsqueeze(1)
        x = x + means @ w["l0.up"].T + plain.mlp(h, {k.replace("l0.", "p.mlp."): v for k, v in w.items()}, "p.")
        h = plain.layer_norm(x, w["l1.ln.weight"], w["l1.ln.bias"], eps)
        wd = {k.replace("l1.", "p."): v for k, v in w.items() if k.startswith("l1.attn")}
        wd.update({k.replace("l1.", "p.mlp."): v for k, v in w.items() if k.startswith("l1.fc")})
        x = x + plain.attention(h, wd, "p.", {"n_heads": 2, "n_kv_heads": 1, "head_dim": 16}, positions,
                                plain.visibility(positions, None), plain.rotary_table(8, 96, 100.0)) + plain.mlp(h, wd, "p.")
        return plain.layer_norm(x, w["fn.weight"], w["fn.bias"], eps) @ w["emb"].T

    lengths = {"a": 50, "b": 21, "c": 38, "d": 45}
    reqs = {tag: helpers.Request(tag, helpers.random_ids(70 + i, n, vocab)) for i, (tag, n) in enumerate(lengths.items())}
    steps = [[("a", 20), ("b", 3)], [("a", 1), ("b", 17), ("c", 30)], [("a", 29), ("b", 1), ("c", 1)],    # a and b end
             [("c", 7), ("d", 33)], [("d", 1)], [("d", 11)]]        # d runs in pages a and b gave back (9 pages in all)
    got = helpers.replay(runner, reqs, steps, poison=True)
    for tag, req in reqs.items():
        helpers.assert_close(got[tag], reference(req.ids), torch.float32, f"latent cache, request {tag}")
    assert all(g.pool.free_count == 9 for g in cache.groups)


def test_a_layer_may_read_another_layers_cache():
    """Schedule entry 1 keeps no keys and values and reads those of entry 0."""
    from kestrel_amd.config import get_spec
    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.parts import ScheduleEntry
    from dataclasses import replace

    spec = get_spec("moondream2")
    plan = spec.build_plan(spec.read_config(helpers.TINY_A))
    plan = replace(plan, schedule=(ScheduleEntry(0), ScheduleEntry(1, reads_cache_of=0)))
    model = DecoderModel(plan)
    weights = {k: v.float() for k, v in helpers.stored_weights(helpers.model_dir("A")).items()}
    model.bind(weights, torch.float32, DEV)
    runner = make_runner(model, 16, 8, 2)
    assert len(runner.cache.groups[0].entries) == 1            # one cache for both runs
    ids = helpers.random_ids(40, 20, 512)
    slot = runner.admit()
    whole = runner.step([StepEntry(slot, ids, want=list(range(20)))]).clone()
    runner.release(slot)
    slot = runner.admit()
    parts = [runner.step([StepEntry(slot, ids[:13], want=list(range(13)))]).clone()]
    parts += [runner.step([StepEntry(slot, [t], want=[0])]).clone() for t in ids[13:]]
    helpers.assert_close(torch.cat(parts), whole, torch.float32, "shared cache: portions against whole")
    # and it equals the plain model whose second layer attends to the first layer's keys and values
    cfg = helpers.flat_config("A")
    w = {k: v.double() for k, v in weights.items()}
    x = w["text.wte"][torch.tensor(ids)]
    positions = torch.arange(20)
    allowed = plain.visibility(positions, None)
    table = plain.rotary_table(plain.rotary_dim_of(cfg), 20, cfg["rope_theta"])
    hd, nh = plain.head_dim_of(cfg), cfg["n_heads"]
    kv0 = None
    for i in range(2):
        p = f"text.blocks.{i}."
        xn = plain.layer_norm(x, w[p + "ln.weight"], w[p + "ln.bias"], plain.eps_of(cfg))
        qkv = plain.linear(xn, w[p + "attn.qkv.weight"], w[p + "attn.qkv.bias"])
        q, k, v = qkv.split([nh * hd, nh * hd, nh * hd], dim=-1)
        q = plain.apply_rotary(q.reshape(20, nh, hd), positions, table)
        if i == 0:
            kv0 = (plain.apply_rotary(k.reshape(20, nh, hd), positions, table), v.reshape(20, nh, hd))
        o = plain.attention_core(q, kv0[0], kv0[1], allowed, hd ** -0.5).reshape(20, nh * hd)
        x = x + plain.linear(o, w[p + "attn.proj.weight"], w[p + "attn.proj.bias"]) + plain.mlp(xn, w, p)
    helpers.assert_close(whole, plain.head(x, w, cfg), torch.float32, "shared cache against plain")


def test_constants_around_the_stack():
    """A plan may scale the looked-up embeddings (not the given ones), scale the logits and cap them
    with a tanh: a tiny Moondream plan with all three against the plain model with the embedding
    table scaled by hand and the logits adjusted by formula; eagerly and as a replayed graph."""
    from kestrel_amd.config import get_spec
    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry
    from kestrel_amd.models import DecoderModel
    from dataclasses import replace

    spec = get_spec("moondream2")
    base = spec.build_plan(spec.read_config(helpers.TINY_A))
    plan = replace(base, embedding_scale=3.0, logit_scale=0.5, logit_softcap=2.0)
    model = DecoderModel(plan)
    weights = {k: v.float() for k, v in helpers.stored_weights(helpers.model_dir("A")).items()}
    model.bind(weights, torch.float32, DEV)
    cfg = helpers.flat_config("A")
    ids = helpers.random_ids(41, 24, cfg["vocab_size"])
    given = torch.randn(5, cfg["dim"], generator=torch.Generator().manual_seed(42))
    w = {k: v.double() for k, v in weights.items()}
    w[plan.names["embedding"]] = w[plan.names["embedding"]] * 3.0
    expected = plain.forward(cfg, w, ids, prefix_embeds=given.double())
    expected = 2.0 * torch.tanh(expected * 0.5 / 2.0)
    for graphs in (False, True):
        runner = make_runner(model, 16, 8, 2, enable_graphs=graphs)
        slot = runner.admit()
        n = 5 + len(ids)
        first = runner.step([StepEntry(slot, [-1] * 5 + ids[:10], want=list(range(15)), embeds=given.to(DEV),
                                       bidirectional=[(0, 5)])]).clone()
        rest = [runner.step([StepEntry(slot, [t], want=[0])]).clone() for t in ids[10:]]
        helpers.assert_close(torch.cat([first] + rest), expected[:n], torch.float32, f"constants around the stack, graphs={graphs}")
        runner.release(slot)


@dataclass(frozen=True)
class GatedSpec:
    kind: str
    dim: int
    hidden_dim: int


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_a_gated_feed_forward_as_a_part(dtype):
    """Another feed-forward, defined here: ``down(silu(x Wg^T) * (x Wu^T))``, three matrices without biases. It
    binds gate and value as one matrix of row pairs and offers its stages like the dense one, so the product
    of the pair is taken in the epilogue of whatever kernel runs its first linear: the prompt's tiled kernel,
    and in decode steps the launch that also normalises and projects q|k|v (one launch for norm + q|k|v + gate
    and value, one for attention, one for both last linears). A tiny Moondream plan with it in every layer
    against a plain computation; prompt portions, then tokens one by one, eagerly and replayed; then prompt portions
    replayed as well, which the part allows by saying ``replays_every_step``."""
    from dataclasses import replace

    from kestrel_amd.config import get_spec
    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.ops.linear import ACT_GATED, activation_code, linear, linear_gated, pair_rows
    from kestrel_amd.parts import FeedForward, ParamSpec, register_feed_forward

    class GatedFeedForward(FeedForward):
        replays_every_step = True      # (its scratch comes from the batch's workspace, and it asks the host side of a batch nothing)

        def params(self):
            d, f = self.spec.dim, self.spec.hidden_dim
            return {"gate.weight": ParamSpec((f, d)), "up.weight": ParamSpec((f, d)), "down.weight": ParamSpec((d, f))}

        def bind(self, tensors, dtype, device):
            self.dtype = dtype
            self.pairs = pair_rows(tensors["gate.weight"].to(device), tensors["up.weight"].to(device))
            self.down = tensors["down.weight"].to(device).contiguous()
            self.act = activation_code("silu")

        def input_projection(self):
            return self.pairs, None, self.spec.hidden_dim, self.act | ACT_GATED

        def output_projection(self):
            return self.down, None

        def forward(self, h, batch, residual):
            hidden = batch.workspace.get("toy.gated_hidden", (h.shape[0], self.spec.hidden_dim), self.dtype)
            linear_gated(h, self.pairs, None, hidden, self.act)
            linear(hidden, self.down, None, residual, accumulate=True)

    register_feed_forward("toy_gated", GatedFeedForward)
    name = "D"
    cfg = helpers.flat_config(name)
    hidden_dim = 72
    spec = get_spec("moondream2")
    base = spec.build_plan(spec.read_config(helpers.CONFIGS[name]))
    layers = []
    for index, layer in enumerate(base.layers):
        names = {k: v for k, v in layer.names.items() if not k.startswith("feed_forward.")}
        names.update({f"feed_forward.{part}.weight": f"text.blocks.{index}.glu.{part}.weight" for part in ("gate", "up", "down")})
        layers.append(replace(layer, feed_forward=GatedSpec("toy_gated", cfg["dim"], hidden_dim), names=names))
    model = DecoderModel(replace(base, layers=tuple(layers)))
    gen = torch.Generator().manual_seed(61)
    stored = helpers.stored_weights(helpers.model_dir(name))
    weights = {}
    for tensor_name, pspec in model.params().items():
        if tensor_name in stored:
            weights[tensor_name] = stored[tensor_name].float()
        else:
            weights[tensor_name] = (0.3 * torch.randn(pspec.shape, generator=gen)).to(dtype).float()
    model.bind({k: v.to(dtype) if v.dim() == 2 else v for k, v in weights.items()}, dtype, DEV)

    ids = helpers.random_ids(62, 45, cfg["vocab_size"])
    w = {k: v.double() for k, v in weights.items()}
    x = w["text.wte"][torch.tensor(ids)]
    positions = torch.arange(len(ids))
    allowed = plain.visibility(positions, None)
    table = plain.rotary_table(plain.rotary_dim_of(cfg), len(ids), float(cfg["rope_theta"]))
    for index in range(cfg["n_layers"]):
        prefix = f"text.blocks.{index}."
        xn = plain.layer_norm(x, w[prefix + "ln.weight"], w[prefix + "ln.bias"], plain.eps_of(cfg))
        gated = torch.nn.functional.silu(xn @ w[prefix + "glu.gate.weight"].T) * (xn @ w[prefix + "glu.up.weight"].T)
        x = x + plain.attention(xn, w, prefix, cfg, positions, allowed, table) + gated @ w[prefix + "glu.down.weight"].T
    expected = plain.head(x, w, cfg)
    for graphs in (False, True):
        runner = make_runner(model, 16, 8, 2, enable_graphs=graphs)
        slot = runner.admit()
        got = [runner.step([StepEntry(slot, ids[:21], want=list(range(21)))]).clone(),
               runner.step([StepEntry(slot, ids[21:30], want=list(range(9)))]).clone()]
        got += [runner.step([StepEntry(slot, [t], want=[0])]).clone() for t in ids[30:]]
        assert (runner.graph_replays > 0) == graphs
        helpers.assert_close(torch.cat(got), expected, dtype, f"a gated feed-forward, graphs={graphs}")
        runner.release(slot)
    # the part says it can be replayed in steps of any shape, the parts around it do too: portions of a prompt of which
    # the scheduler's places are wanted go through the graph of their bucket of tokens
    runner = make_runner(model, 16, 8, 2, enable_graphs=True)
    assert runner.mixed_graphs
    slot = runner.admit()
    got = [runner.step([StepEntry(slot, ids[:21], want=[20])]).clone(), runner.step([StepEntry(slot, ids[21:30], want=[7, 8])]).clone()]
    assert runner.mixed_graph_replays == 2 and sorted(runner._mixed) == [(16, 2), (32, 2)]
    helpers.assert_close(torch.cat(got), expected[[20, 28, 29]], dtype, "a gated feed-forward in replayed prompt steps")
    runner.release(slot)
    if dtype == torch.bfloat16:
        # the decode steps took the three-launch form: the gated linear rode in the launch of norm + q|k|v, or
        # (a few rows whose attention leaves the chip idle) in the attention launch
        from kestrel_amd.ops import fast
        rode = []
        first_launch, attention_launch = fast.layernorm_linear, fast.attention_decode_bf16

        def watched_first(*args, **kwargs):
            done = first_launch(*args, **kwargs)
            rode.append(done and len(args) > 11 and args[11])
            return done

        def watched_attention(*args, **kwargs):
            done = attention_launch(*args, **kwargs)
            rode.append(done and kwargs.get("beside") is not None and kwargs["beside"].act)
            return done

        fast.layernorm_linear, fast.attention_decode_bf16 = watched_first, watched_attention
        try:
            runner = make_runner(model, 16, 8, 2)
            slot = runner.admit()
            runner.step([StepEntry(slot, ids[:5])])
            runner.step([StepEntry(slot, ids[5:6], want=[0])])
        finally:
            fast.layernorm_linear, fast.attention_decode_bf16 = first_launch, attention_launch
        # (both steps have few rows: the prompt's five tokens take the same three launches a layer)
        assert rode.count(activation_code("silu") | ACT_GATED) == 2 * cfg["n_layers"], rode


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_another_norm_as_a_part(dtype):
    """Another norm, defined here: ``x / sqrt(mean(x^2) + eps) * weight`` (no mean taken off, no shift), in every
    block and before the head of a tiny Moondream plan. It does not claim to be a LayerNorm
    (``layernorm_operands`` stays ``None``), so no kernel takes it into its launch: blocks and head run it through
    its ``forward``, also in decode steps and under replayed graphs. Against a plain computation."""
    from dataclasses import replace

    from kestrel_amd.config import get_spec
    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.parts import Norm, NormSpec, ParamSpec, register_norm

    class RootMeanSquare(Norm):
        def params(self):
            return {"weight": ParamSpec((self.spec.dim,), "vector", "gain")}

        def bind(self, tensors, dtype, device):
            self.weight = tensors["weight"].to(device=device, dtype=torch.float32)

        def forward(self, x, out, rows=None):
            picked = x if rows is None else x[rows.long()]
            out.copy_(picked * torch.rsqrt(picked.pow(2).mean(dim=-1, keepdim=True) + self.spec.eps) * self.weight)

    register_norm("toy_rms", RootMeanSquare)
    name = "D"
    cfg = helpers.flat_config(name)
    spec = get_spec("moondream2")
    base = spec.build_plan(spec.read_config(helpers.CONFIGS[name]))
    rms = NormSpec("toy_rms", cfg["dim"], 1e-5, bias=False)
    layers = tuple(replace(layer, norm=rms, names={k: v for k, v in layer.names.items() if k != "norm.bias"})
                   for layer in base.layers)
    plan = replace(base, layers=layers, final_norm=rms, names={k: v for k, v in base.names.items() if k != "final_norm.bias"})
    model = DecoderModel(plan)
    weights = {k: v.float() for k, v in helpers.stored_weights(helpers.model_dir(name)).items() if k in model.params()}
    assert set(weights) == set(model.params())
    model.bind({k: v.to(dtype) if v.dim() == 2 else v for k, v in weights.items()}, dtype, DEV)

    def rms_norm(x, weight):
        return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + 1e-5) * weight

    ids = helpers.random_ids(71, 40, cfg["vocab_size"])
    w = {k: v.double() for k, v in weights.items()}
    x = w["text.wte"][torch.tensor(ids)]
    positions = torch.arange(len(ids))
    allowed = plain.visibility(positions, None)
    table = plain.rotary_table(plain.rotary_dim_of(cfg), len(ids), float(cfg["rope_theta"]))
    for index in range(cfg["n_layers"]):
        prefix = f"text.blocks.{index}."
        xn = rms_norm(x, w[prefix + "ln.weight"])
        x = x + plain.attention(xn, w, prefix, cfg, positions, allowed, table) + plain.mlp(xn, w, prefix)
    expected = plain.linear(rms_norm(x, w["text.post_ln.weight"]), w["text.lm_head.weight"], w["text.lm_head.bias"])
    for graphs in (False, True):
        runner = make_runner(model, 16, 8, 2, enable_graphs=graphs)
        slot = runner.admit()
        got = [runner.step([StepEntry(slot, ids[:26], want=list(range(26)))]).clone()]
        got += [runner.step([StepEntry(slot, [t], want=[0])]).clone() for t in ids[26:]]
        assert (runner.graph_replays > 0) == graphs
        helpers.assert_close(torch.cat(got), expected, dtype, f"another norm, graphs={graphs}")
        runner.release(slot)


@dataclass(frozen=True)
class GridPositionSpec:
    kind: str
    dim: int
    rows: int
    columns: int


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_a_position_encoding_of_the_whole_model_over_two_axes(dtype):
    """Another position encoding, defined here: two learned tables, one per axis (row and column), whose
    vectors are added to the embeddings before the first block. It says ``axes = 2``; the step then carries
    two numbers per token: what an entry gives (an image's patches as a grid), else the place in the
    sequence on both axes (text, decoded tokens). A tiny Moondream plan with it (the attention keeps its
    rotation by the place in the sequence) against the plain model fed with embeddings that have the
    position vectors added by hand; a prompt in portions, then tokens one by one, eagerly and replayed."""
    from dataclasses import replace

    from kestrel_amd.config import get_spec
    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.engine.step import StepEntry, StepRefused
    from kestrel_amd.models import DecoderModel
    from kestrel_amd.parts import ParamSpec, PositionEncoding, register_position

    class GridPosition(PositionEncoding):
        axes = 2

        def params(self):
            return {"rows": ParamSpec((self.spec.rows, self.spec.dim), "matrix", "normal"),
                    "columns": ParamSpec((self.spec.columns, self.spec.dim), "matrix", "normal")}

        def bind(self, tensors, dtype, device):
            self.rows, self.columns = tensors["rows"].to(device).float(), tensors["columns"].to(device).float()

        def add_to_embeddings(self, x, batch):
            at = batch.position_axes.long()
            x += self.rows[at[:, 0]] + self.columns[at[:, 1]]

    register_position("toy_grid", GridPosition)
    spec = get_spec("moondream2")
    cfg = helpers.flat_config("E")
    base = spec.build_plan(spec.read_config(helpers.TINY_E))
    plan = replace(base, position=GridPositionSpec("toy_grid", cfg["dim"], 64, 64),
                   names={**base.names, "position.rows": "pos.rows", "position.columns": "pos.columns"})
    model = DecoderModel(plan)
    assert model.position_axes() == 2
    stored = helpers.stored_weights(helpers.model_dir("E"))
    gen = torch.Generator().manual_seed(51)
    weights = {k: v.float() for k, v in stored.items()}
    weights["pos.rows"] = 0.5 * torch.randn(64, cfg["dim"], generator=gen)
    weights["pos.columns"] = 0.5 * torch.randn(64, cfg["dim"], generator=gen)
    weights = {k: v.to(dtype).float() for k, v in weights.items()}          # what both sides compute with
    assert set(model.params()) == set(weights)
    model.bind({k: v.to(dtype) if v.dim() == 2 else v for k, v in weights.items()}, dtype, DEV)
    # 6 text ids, a grid of 3 x 4 patches (given embeddings, numbered by row and column), 9 text ids, then decoding
    ids_a, ids_b = helpers.random_ids(52, 6, cfg["vocab_size"]), helpers.random_ids(53, 9 + 6, cfg["vocab_size"])
    patches = torch.randn(12, cfg["dim"], generator=gen)
    grid = [(10 + r, 20 + c) for r in range(3) for c in range(4)]
    numbers = [(p, p) for p in range(6)] + grid + [(p, p) for p in range(18, 18 + len(ids_b))]
    table = weights[plan.names["embedding"]].double()
    embedded = torch.cat([table[ids_a], patches.double(), table[ids_b]])
    embedded = embedded + torch.stack([weights["pos.rows"][r].double() + weights["pos.columns"][c].double() for r, c in numbers])
    block_of = [-1] * 6 + [0] * 12 + [-1] * len(ids_b)
    expected = plain.forward(cfg, {k: v.double() for k, v in weights.items()}, [], prefix_embeds=embedded, block_ids=block_of)
    for graphs in (False, True):
        runner = make_runner(model, 16, 8, 2, enable_graphs=graphs)
        slot = runner.admit()
        with pytest.raises(StepRefused, match=r"shape \[2, 2\]"):
            runner.step([StepEntry(slot, ids_a[:2], positions=[(0, 0, 0), (1, 1, 1)])])
        got = [runner.step([StepEntry(slot, ids_a[:4], want=[0, 1, 2, 3])]).clone()]
        # the rest of the first text and the whole grid in one portion: positions given for all of its tokens
        got.append(runner.step([StepEntry(slot, ids_a[4:] + [-1] * 12, want=list(range(14)), embeds=patches.to(DEV),
                                          bidirectional=[(6, 18)], positions=[(4, 4), (5, 5)] + grid)]).clone())
        got.append(runner.step([StepEntry(slot, ids_b[:9], want=list(range(9)))]).clone())
        got += [runner.step([StepEntry(slot, [t], want=[0])]).clone() for t in ids_b[9:]]
        assert (runner.graph_replays > 0) == graphs
        helpers.assert_close(torch.cat(got), expected, dtype, f"a two-axis position encoding, graphs={graphs}")
        runner.release(slot)
    # an encoding of several axes cannot stand inside attention, which turns by the place in the sequence
    from kestrel_amd.parts import AttentionSpec, build_part

    mixer = build_part("mixer", AttentionSpec("attention", 32, 2, 2, 16, GridPositionSpec("toy_grid", 32, 4, 4)))
    with pytest.raises(ValueError, match="takes 2 numbers per token"):
        mixer.bind({name: torch.zeros(p.shape) for name, p in mixer.params().items()}, torch.float32, DEV)


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "replayed"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_a_windowed_layer_beside_a_full_one(dtype, graphs):
    """The second layer of a tiny Moondream plan is given a window of 24 keys: its keys and values
    live in a group with a pool of its own, which gives pages back as the window passes them, while
    the first layer keeps all keys. Two requests in portions and single tokens, against the plain
    model with the window in the second layer's mask. Replayed: every step is a graph (of decode rows or
    of a bucket of tokens), whose padding tokens have a window's start of their own; only the last place
    of every portion is wanted then."""
    from dataclasses import replace

    from kestrel_amd.config import get_spec
    from kestrel_amd.engine.loading import make_runner
    from kestrel_amd.models import DecoderModel
    from tests.helpers import Request

    name, window = "D", 24
    spec = get_spec("moondream2")
    plan = spec.build_plan(spec.read_config(helpers.CONFIGS[name]))
    layers = list(plan.layers)
    layers[1] = replace(layers[1], mixer=replace(layers[1].mixer, window=window))
    model = DecoderModel(replace(plan, layers=tuple(layers)))
    stored = helpers.stored_weights(helpers.model_dir(name))
    model.bind(dict(stored), dtype, DEV)
    runner = make_runner(model, 16, 12, 2, enable_graphs=graphs)
    assert len(runner.cache.groups) == 2 and [g.spec.window for g in runner.cache.groups] == [None, window]
    helpers.poison_cache(runner)
    cfg = helpers.flat_config(name)
    reqs = {"a": Request("a", helpers.random_ids(60, 100, cfg["vocab_size"])),
            "b": Request("b", helpers.random_ids(61, 58, cfg["vocab_size"]))}
    steps = [[("a", 37)], [("a", 30), ("b", 20)], [("a", 1), ("b", 33)]] + [[("a", 1), ("b", 1)] for _ in range(5)] \
        + [[("a", 1)] for _ in range(27)]
    held = []
    original = runner.step

    def step_and_count(entries):
        out = original(entries)
        held.append(runner.cache.n_pages - runner.cache.groups[1].pool.free_count)
        return out

    runner.step = step_and_count
    if graphs:
        from tests.test_mixed_graphs_gpu import replay_last_places
        places = replay_last_places(runner, reqs, steps, wanted=1)
        assert runner.mixed_graph_replays == 3 and runner.graph_replays == len(steps) - 3
    else:
        got = helpers.replay(runner, reqs, steps, poison=True)
    # the windowed group never holds more than the window and a portion's worth of pages per request
    assert max(held) <= 2 * (-(-(window + 37) // 16) + 1) and held[-1] <= -(-window // 16) + 1
    assert all(g.pool.free_count == runner.cache.n_pages for g in runner.cache.groups)
    for tag, req in reqs.items():
        n = req.length
        w = {k: v.double() for k, v in stored.items()}
        x = w["text.wte"][torch.tensor(req.ids)]
        positions = torch.arange(n)
        causal = plain.visibility(positions, None)
        near = causal & (positions.unsqueeze(1) - positions.unsqueeze(0) < window)
        table = plain.rotary_table(plain.rotary_dim_of(cfg), n, cfg["rope_theta"])
        x = plain.block(x, w, 0, cfg, positions, causal, table)
        x = plain.block(x, w, 1, cfg, positions, near, table)
        expected = plain.head(x, w, cfg)
        if graphs:
            at = sorted(places[tag])
            helpers.assert_close(torch.stack([places[tag][p] for p in at]), expected[at], dtype, f"windowed layer replayed, request {tag}")
        else:
            helpers.assert_close(got[tag], expected, dtype, f"windowed layer, request {tag}")
