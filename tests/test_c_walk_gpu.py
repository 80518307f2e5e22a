"""The C side of a step takes parts by registry: a mixer that the framework has never heard of,
defined here with a HIP kernel and a runner of its own (``tests/toy_parts/running_mean.hip``),
is registered, built into a toy architecture and stepped through ``kappai_forward`` without a
change to the framework's files, bit for bit equal to the same steps run part by part from the
host; and what has no description for the C side runs from the host as before.  The same for a
norm and an arrangement of parts from outside (``tests/toy_parts/layer_norm_block.hip``:
LayerNorm, and a block whose mixer and feed-forward read the same normalised rows) around the
framework's own mixers and feed-forward, and for an encoding of positions that is added to the
embedded rows (``tests/toy_parts/learned_positions.hip``)."""
import ctypes
from ctypes import Structure, c_int, c_void_p
from dataclasses import dataclass
from pathlib import Path

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOY_SOURCE = Path(__file__).resolve().parent / "toy_parts" / "running_mean.hip"
TOY_BLOCK_SOURCE = Path(__file__).resolve().parent / "toy_parts" / "layer_norm_block.hip"
TOY_POSITIONS_SOURCE = Path(__file__).resolve().parent / "toy_parts" / "learned_positions.hip"


def toy_library():
    from kappai_amd.kernels.lib import library_at
    lib = library_at(TOY_SOURCE)
    lib.toy_running_mean_run.restype = None       # only its address is used
    return lib


def define_toy():
    """Registers the toy mixer and the toy architecture (once) and returns the mixer's class."""
    from kappai_amd.cache import FixedState
    from kappai_amd.config import ModelConfig, register_architecture
    from kappai_amd.kernels import ops
    from kappai_amd.models import LayerCall, Model
    from kappai_amd.parts import Linear, Mixer, OutputHead, TokenEmbedding, make_part, register_part
    from kappai_amd.parts.cdesc import RUNNER_PART, LinearDesc

    from kappai_amd.parts import MIXERS
    if "toy_running_mean_hip" in MIXERS:
        return MIXERS["toy_running_mean_hip"]

    class ToyDesc(Structure):
        """``toy_running_mean`` of tests/toy_parts/running_mean.hip."""
        _fields_ = [("proj", LinearDesc), ("state", c_void_p)]

    class RunningMeanHip(Mixer):
        """out_t = W * mean(x_0 .. x_t); state [width] float32: the running sum."""

        def __init__(self, prefix, width, dtype):
            self.width, self.dtype = width, dtype
            self.proj = Linear([prefix + "proj"], width, [width])

        def cache_spec(self):
            return FixedState((self.width,), "float32")

        def tensor_specs(self):
            return self.proj.tensor_specs()

        def bind(self, tensors):
            self.proj.bind(tensors)

        def forward(self, x, batch, cache, shared_cache=False):
            lib = toy_library()
            mean = torch.empty((x.shape[0], self.width), dtype=x.dtype, device=x.device)
            rc = lib.toy_running_mean_launch(
                c_void_p(x.data_ptr()), c_int(x.stride(0)), c_void_p(mean.data_ptr()),
                c_void_p(cache.state.data_ptr()), c_void_p(batch.seg_start.data_ptr()),
                c_void_p(batch.seg_pos0.data_ptr()), c_void_p(batch.seg_slot.data_ptr()),
                c_int(batch.n_segments), c_int(self.width),
                c_int(1 if x.dtype == torch.bfloat16 else 0), ops._stream())
            assert rc == 0, rc
            return self.proj.forward(mean)

        def c_part(self, plan, view, shared_cache=False):
            lib = toy_library()
            assert lib.toy_running_mean_desc_bytes() == ctypes.sizeof(ToyDesc)
            plan.register_runner("mixer.toy_running_mean", RUNNER_PART, lib.toy_running_mean_run,
                                 ToyDesc)
            first = plan.linear(self.proj)
            return plan.part("mixer.toy_running_mean", ToyDesc(first, view.state.data_ptr()))

    register_part("mixer", "toy_running_mean_hip", RunningMeanHip)

    class ChangedForward(RunningMeanHip):
        """A subclass that changes ``forward`` and says nothing about C: twice the mean."""

        def forward(self, x, batch, cache, shared_cache=False):
            return 2 * super().forward(x, batch, cache, shared_cache)

    register_part("mixer", "toy_running_mean_changed", ChangedForward)

    @dataclass
    class ToyConfig(ModelConfig):
        width: int = 0
        vocab_size: int = 0
        heads: int = 0
        head_dim: int = 0
        ff: int = 0
        eps: float = 1e-5
        mixer: str = "toy_running_mean_hip"
        max_position_embeddings: int = 512

        @classmethod
        def from_dict(cls, raw):
            return cls(architecture="ToyHipForCausalLM", **{k: raw[k] for k in
                       ("width", "vocab_size", "heads", "head_dim", "ff", "eps", "mixer")})

        def to_dict(self):
            return {"architectures": ["ToyHipForCausalLM"], "width": self.width,
                    "vocab_size": self.vocab_size, "heads": self.heads, "head_dim": self.head_dim,
                    "ff": self.ff, "eps": self.eps, "mixer": self.mixer}

    def build_toy(cfg, dtype):
        def norm(name):
            return make_part("norm", "rmsnorm", name=name, width=cfg.width, eps=cfg.eps,
                             dtype=dtype)

        def block(i, mixer):
            p = f"blocks.{i}."
            return make_part("block", "pre_norm", mixer_norm=norm(p + "n1"), mixer=mixer,
                             ffn_norm=norm(p + "n2"),
                             feed_forward=make_part("feed_forward", "swiglu", prefix=p + "ff.",
                                                    width=cfg.width, hidden=cfg.ff, dtype=dtype))
        rot = make_part("position_encoding", "rotary", head_dim=cfg.head_dim, theta=100.0)

        def attn(i):
            return make_part("mixer", "attention", prefix=f"blocks.{i}.att.", width=cfg.width,
                             num_heads=cfg.heads, num_kv_heads=cfg.heads // 2,
                             head_dim=cfg.head_dim, dtype=dtype, position=rot, qk_norm_eps=1e-5)
        layers = [block(0, make_part("mixer", cfg.mixer, prefix="blocks.0.mix.", width=cfg.width,
                                     dtype=dtype)),
                  block(1, attn(1)), block(2, attn(2))]
        emb = TokenEmbedding("emb", cfg.vocab_size, cfg.width)
        # block 0 runs twice (two states), block 2 reads the keys that block 1 stored
        schedule = [LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(2, reads_cache_of=1)]
        return Model(cfg, dtype, emb, layers, norm("final"),
                     OutputHead("head", cfg.vocab_size, cfg.width, tied_to=emb), schedule=schedule)

    register_architecture("ToyHipForCausalLM", ToyConfig, build_toy)
    return RunningMeanHip


TOY = {"architectures": ["ToyHipForCausalLM"], "width": 64, "vocab_size": 211, "heads": 4,
       "head_dim": 32, "ff": 96, "eps": 1e-5, "mixer": "toy_running_mean_hip"}


def toy_model(tmp_path, dtype, mixer="toy_running_mean_hip"):
    from kappai_amd.config import config_from_dict
    from kappai_amd.models import load_model
    from kappai_amd.weights import write_random_model
    define_toy()
    folder = tmp_path / f"toy_{mixer}"
    if not folder.exists():
        write_random_model(folder, config_from_dict(dict(TOY, mixer=mixer)), seed=5, std=0.2,
                           norm_jitter=0.1)
    return load_model(folder, dtype, DEV)


def replay(model, steps, peak, out_dir, c_forward, graphs):
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    cache = make_replay_cache(model, peak)
    cache.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cache, DEV, decode_graphs=graphs, c_forward=c_forward)
    rep = TraceReplayer(runner, out_dir)
    results = [rep.run_step(obj) for obj in steps]
    cache.check()
    return results, runner


def test_the_toy_kernel_is_a_running_mean():
    """The toy's kernel against torch: a portion after a history (the sum so far in the state),
    a fresh request beside it (whatever the slot held before is not read)."""
    lib = toy_library()
    D = 70
    x = torch.randn(9, D, generator=torch.Generator().manual_seed(1))
    state = torch.full((3, D), float("nan"))
    history = torch.randn(4, D, generator=torch.Generator().manual_seed(2))
    state[2] = history.sum(0)
    seg_start = torch.tensor([0, 5, 9], dtype=torch.int32, device=DEV)
    seg_pos0 = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    seg_slot = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
    xd, sd = x.to(DEV), state.to(DEV)
    out = torch.empty_like(xd)
    rc = lib.toy_running_mean_launch(
        c_void_p(xd.data_ptr()), c_int(D), c_void_p(out.data_ptr()), c_void_p(sd.data_ptr()),
        c_void_p(seg_start.data_ptr()), c_void_p(seg_pos0.data_ptr()),
        c_void_p(seg_slot.data_ptr()), c_int(2), c_int(D), c_int(0),
        c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    want = torch.cat([(history.sum(0) + torch.cumsum(x[:5], 0)) / torch.arange(5, 10)[:, None],
                      torch.cumsum(x[5:], 0) / torch.arange(1, 5)[:, None]])
    assert float((out.cpu() - want).abs().max()) < 1e-5
    assert float((sd[2].cpu() - (history.sum(0) + x[:5].sum(0))).abs().max()) < 1e-5
    assert float((sd[0].cpu() - x[5:].sum(0)).abs().max()) < 1e-5
    assert torch.isnan(sd[1]).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_from_outside_runs_from_c(tmp_path, dtype):
    """The toy architecture (the toy mixer run twice with two states, attention, an attention
    call that reads another call's keys) under the mixed schedule: launched from C it gives bit
    for bit what the host's part-by-part walk gives, with and without decode graphs, and the
    portions give what whole prompts give."""
    import schedules
    from replay_common import collect, make_requests
    model = toy_model(tmp_path, dtype)
    requests = make_requests(TOY["vocab_size"], [70, 45, 100, 37, 83, 64, 29], seed=22)
    steps, index, peak = schedules.mixed(requests)
    results = {}
    for c_forward in (True, False):
        for graphs in (False, True):
            res, runner = replay(model, steps, peak, tmp_path / f"c{c_forward}g{graphs}",
                                 c_forward, graphs)
            assert (runner._cplan is not None) == c_forward, "the toy model has a description"
            if graphs:
                assert runner.graph_replays > 0
            results[(c_forward, graphs)] = res
    base = results[(False, False)]
    for key, res in results.items():
        for a, b in zip(base, res):
            assert (a is None) == (b is None)
            if a is not None:
                assert np.array_equal(a, b), key
    # and cut into portions it is the model that whole prompts give
    whole_steps, whole_index, whole_peak = schedules.whole(requests)
    whole, _ = replay(model, whole_steps, whole_peak, tmp_path / "whole", True, False)
    got = collect(index, {s["step"]: r for s, r in zip(steps, base) if r is not None},
                  TOY["vocab_size"])
    ref = collect(whole_index, {s["step"]: r for s, r in zip(whole_steps, whole) if r is not None},
                  TOY["vocab_size"])
    scale = max(float(np.abs(v).max()) for v in ref.values())
    tol = 2e-5 if dtype == "float32" else 4e-2
    worst = max(float(np.abs(got[k] - ref[k]).max()) for k in ref) / scale
    assert worst < tol, worst


def test_the_toy_mixer_does_what_it_says_inside_the_model(tmp_path):
    """With every other part's contribution removed (out projections and down projections zero),
    the logits are head(norm(embedding + W mean(norm(embedding)) twice over)): worked out in
    float64 from the weights, against the C walk."""
    model = toy_model(tmp_path, "float32")
    for blk in model.layers:
        blk.feed_forward.down.weight.zero_()
        if hasattr(blk.mixer, "out"):
            blk.mixer.out.weight.zero_()
    toks = [int(t) for t in np.random.default_rng(3).integers(0, TOY["vocab_size"], size=19)]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks, "want": list(range(19))}],
              "end": ["a"]}]
    (got,), runner = replay(model, steps, 64, tmp_path / "zeroed", True, False)
    assert runner._cplan is not None
    E = model.embedding.table.double().cpu().numpy()
    blk = model.layers[0]
    W = blk.mixer.proj.weight.double().cpu().numpy()
    n1 = blk.mixer_norm.weight.double().cpu().numpy()
    fin = model.final_norm.weight.double().cpu().numpy()

    def rms(x, w):
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + TOY["eps"]) * w
    x = E[toks]
    for _ in range(2):                       # block 0 runs twice
        xb = rms(x, n1)
        x = x + (np.cumsum(xb, 0) / np.arange(1, 20)[:, None]) @ W.T
    want = rms(x, fin) @ E.T
    assert float(np.abs(got - want).max()) < 2e-5 * float(np.abs(want).max())


def test_a_part_that_changed_forward_without_a_description_runs_from_the_host(tmp_path):
    """A subclass of the toy mixer changes ``forward`` and gives no description of its own: it
    must not inherit its parent's runner.  Its model runs part by part from the host, and its
    logits differ from the parent's."""
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [5, 9, 200, 17, 3], "want": [4]}],
              "end": ["a"]}]
    changed = toy_model(tmp_path, "float32", mixer="toy_running_mean_changed")
    (got,), runner = replay(changed, steps, 64, tmp_path / "changed", True, False)
    assert runner._cplan is None
    parent = toy_model(tmp_path, "float32")
    (base,), runner = replay(parent, steps, 64, tmp_path / "parent", True, False)
    assert runner._cplan is not None
    assert float(np.abs(got - base).max()) > 1e-3


def test_runners_are_looked_up_by_name_and_checked():
    """The registry: the framework's own parts are there under their names; an unknown name and
    a description of another size are refused with a message."""
    from kappai_amd.engine.cforward import engine_library
    from kappai_amd.kernels.lib import KernelLaunchError
    from kappai_amd.parts.cdesc import RUNNER_NORM, RUNNER_PART, CPlan, FoldDesc, LinearDesc

    plan = CPlan(engine_library(), type("M", (), {"dtype": torch.float32})(), None, DEV)
    assert plan.runner("norm.rms", RUNNER_NORM, FoldDesc)
    with pytest.raises(KernelLaunchError, match="no runner is registered"):
        plan.runner("mixer.nobody", RUNNER_PART, FoldDesc)
    with pytest.raises(KernelLaunchError, match="no runner is registered"):
        plan.runner("norm.rms", RUNNER_PART, FoldDesc)            # another kind
    with pytest.raises(KernelLaunchError, match="reads a description of"):
        plan.runner("mixer.conv", RUNNER_PART, LinearDesc)
    lib = toy_library()
    plan.register_runner("mixer.toy_again", RUNNER_PART, lib.toy_running_mean_run, FoldDesc)
    plan.register_runner("mixer.toy_again", RUNNER_PART, lib.toy_running_mean_run, FoldDesc)
    with pytest.raises(KernelLaunchError, match="registered already"):
        plan.register_runner("mixer.toy_again", RUNNER_PART, lib.toy_running_mean_launch, FoldDesc)


# ---------------------------------------------------------------------------------------------
# a norm and a block from outside
# ---------------------------------------------------------------------------------------------
def toy_block_library():
    from kappai_amd.kernels.lib import library_at
    lib = library_at(TOY_BLOCK_SOURCE)
    lib.toy_layer_norm_run.restype = None         # only their addresses are used
    lib.toy_parallel_block_run.restype = None
    return lib


def define_toy_block():
    """Registers the toy norm, the toy block and an architecture made of them (once)."""
    from kappai_amd.config import ModelConfig, register_architecture
    from kappai_amd.kernels import ops
    from kappai_amd.models import Model
    from kappai_amd.parts import (NORMS, Block, Hidden, Norm, OutputHead, TokenEmbedding,
                                  make_part, register_part)
    from kappai_amd.parts.base import summed_delta
    from kappai_amd.parts.cdesc import (RUNNER_BLOCK, RUNNER_NORM, NormPartDesc, PartDesc,
                                        defined_together)
    from kappai_amd.weights.spec import INIT_ONES, INIT_SMALL, VECTOR, TensorSpec
    if "toy_layer_norm" in NORMS:
        return

    class LayerNormDesc(Structure):
        """``toy_layer_norm`` of tests/toy_parts/layer_norm_block.hip."""
        _fields_ = [("w", c_void_p), ("b", c_void_p), ("eps", ctypes.c_float)]

    class ParallelBlockDesc(Structure):
        """``toy_parallel_block`` of tests/toy_parts/layer_norm_block.hip."""
        _fields_ = [("norm", NormPartDesc), ("mixer", PartDesc), ("feed_forward", PartDesc)]

    class ToyLayerNorm(Norm):
        """``(x - mean) / sqrt(var + eps) * w + b``; adds the update into the stream first."""

        def __init__(self, name, width, eps, dtype):
            self.name, self.width, self.eps, self.dtype = name, width, float(eps), dtype

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.width,), VECTOR, INIT_ONES),
                    TensorSpec(self.name + ".bias", (self.width,), VECTOR, INIT_SMALL)]

        def bind(self, tensors):
            self.weight = tensors[self.name + ".weight"].to(torch.float32).contiguous()
            self.bias = tensors[self.name + ".bias"].to(torch.float32).contiguous()

        def add_norm(self, resid, delta, rows=None):
            n = resid.shape[0] if rows is None else rows.shape[0]
            out = torch.empty((n, self.width), dtype=self.dtype, device=resid.device)
            kind = 0 if delta is None else 2 if delta.dtype == torch.float32 else 1
            rc = toy_block_library().toy_layer_norm_launch(
                c_void_p(resid.data_ptr()), c_void_p(delta.data_ptr() if delta is not None else 0),
                c_int(kind), c_void_p(self.weight.data_ptr()), c_void_p(self.bias.data_ptr()),
                c_void_p(out.data_ptr()), c_int(1 if self.dtype == torch.bfloat16 else 0),
                c_void_p(rows.data_ptr() if rows is not None else 0), c_int(n), c_int(self.width),
                ctypes.c_float(self.eps), ops._stream())
            assert rc == 0, rc
            return out

        def c_norm(self, plan):
            lib = toy_block_library()
            assert lib.toy_layer_norm_desc_bytes() == ctypes.sizeof(LayerNormDesc)
            plan.register_runner("norm.toy_layer", RUNNER_NORM, lib.toy_layer_norm_run,
                                 LayerNormDesc)
            return plan.norm("norm.toy_layer", LayerNormDesc(self.weight.data_ptr(),
                                                             self.bias.data_ptr(), self.eps))

    register_part("norm", "toy_layer_norm", ToyLayerNorm)

    class ParallelBlock(Block):
        """``h = norm(x); x += mixer(h); x += feed_forward(h)``."""

        def __init__(self, norm, mixer, feed_forward):
            self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward

        def _parts(self):
            return (self.norm, self.mixer, self.feed_forward)

        capturable = True

        def tensor_specs(self):
            return [t for p in self._parts() for t in p.tensor_specs()]

        def bind(self, tensors):
            for p in self._parts():
                p.bind(tensors)

        def weight_bytes(self):
            return sum(p.weight_bytes() for p in self._parts())

        def forward(self, h, batch, cache, shared_cache=False):
            resid = h.resid
            x = self.norm.add_norm(resid, summed_delta(self.norm, h.delta))
            mixed = summed_delta(self.norm, self.mixer.forward(x, batch, cache,
                                                               shared_cache=shared_cache))
            if mixed is not None:
                rc = toy_block_library().toy_add_launch(
                    c_void_p(resid.data_ptr()), c_void_p(mixed.data_ptr()),
                    c_int(1 if mixed.dtype == torch.float32 else 0),
                    ctypes.c_long(mixed.numel()), ops._stream())
                assert rc == 0, rc
            return Hidden(resid, self.feed_forward.forward(x, batch))

        def c_call(self, plan, view, shared_cache=False):
            for part, method, c_method in ((self.norm, "add_norm", "c_norm"),
                                           (self.mixer, "forward", "c_part"),
                                           (self.feed_forward, "forward", "c_part")):
                if not defined_together(part, method, c_method):
                    return None
            lib = toy_block_library()
            assert lib.toy_parallel_block_desc_bytes() == ctypes.sizeof(ParallelBlockDesc)
            plan.register_runner("block.toy_parallel", RUNNER_BLOCK, lib.toy_parallel_block_run,
                                 ParallelBlockDesc)
            norm = self.norm.c_norm(plan)
            mixer = self.mixer.c_part(plan, view, shared_cache)
            feed_forward = self.feed_forward.c_part(plan, None, False)
            if norm is None or mixer is None or feed_forward is None:
                return None
            return plan.call("block.toy_parallel", ParallelBlockDesc(norm, mixer, feed_forward))

    register_part("block", "toy_parallel", ParallelBlock)

    @dataclass
    class ToyBlockConfig(ModelConfig):
        width: int = 0
        vocab_size: int = 0
        heads: int = 0
        head_dim: int = 0
        ff: int = 0
        taps: int = 3
        eps: float = 1e-5
        max_position_embeddings: int = 512

        KEYS = ("width", "vocab_size", "heads", "head_dim", "ff", "taps", "eps")

        @classmethod
        def from_dict(cls, raw):
            return cls(architecture="ToyParallelForCausalLM", **{k: raw[k] for k in cls.KEYS})

        def to_dict(self):
            return {"architectures": ["ToyParallelForCausalLM"],
                    **{k: getattr(self, k) for k in self.KEYS}}

    def build(cfg, dtype):
        def layer_norm(name):
            return make_part("norm", "toy_layer_norm", name=name, width=cfg.width, eps=cfg.eps,
                             dtype=dtype)

        def rms(name):
            return make_part("norm", "rmsnorm", name=name, width=cfg.width, eps=cfg.eps,
                             dtype=dtype)

        def ffn(p):
            return make_part("feed_forward", "swiglu", prefix=p + "ff.", width=cfg.width,
                             hidden=cfg.ff, dtype=dtype)
        rot = make_part("position_encoding", "rotary", head_dim=cfg.head_dim, theta=100.0)

        def attn(p):
            return make_part("mixer", "attention", prefix=p + "att.", width=cfg.width,
                             num_heads=cfg.heads, num_kv_heads=cfg.heads // 2,
                             head_dim=cfg.head_dim, dtype=dtype, position=rot, qk_norm_eps=1e-5)

        def conv(p):
            return make_part("mixer", "conv", prefix=p + "conv.", width=cfg.width,
                             kernel_size=cfg.taps, dtype=dtype, bias=True)
        layers = [
            make_part("block", "toy_parallel", norm=layer_norm("blocks.0.n"), mixer=conv("blocks.0."),
                      feed_forward=ffn("blocks.0.")),
            make_part("block", "pre_norm", mixer_norm=rms("blocks.1.n1"), mixer=attn("blocks.1."),
                      ffn_norm=layer_norm("blocks.1.n2"), feed_forward=ffn("blocks.1.")),
            make_part("block", "toy_parallel", norm=layer_norm("blocks.2.n"), mixer=attn("blocks.2."),
                      feed_forward=ffn("blocks.2.")),
            make_part("block", "pre_norm", mixer_norm=rms("blocks.3.n1"), mixer=conv("blocks.3."),
                      ffn_norm=rms("blocks.3.n2"), feed_forward=ffn("blocks.3.")),
        ]
        emb = TokenEmbedding("emb", cfg.vocab_size, cfg.width)
        return Model(cfg, dtype, emb, layers, layer_norm("final"),
                     OutputHead("head", cfg.vocab_size, cfg.width, tied_to=emb))

    register_architecture("ToyParallelForCausalLM", ToyBlockConfig, build)


TOY_BLOCK = {"architectures": ["ToyParallelForCausalLM"], "width": 96, "vocab_size": 173,
             "heads": 4, "head_dim": 16, "ff": 160, "taps": 3, "eps": 1e-5}


def toy_block_model(tmp_path, dtype):
    from kappai_amd.config import config_from_dict
    from kappai_amd.models import load_model
    from kappai_amd.weights import write_random_model
    define_toy_block()
    folder = tmp_path / "toy_block"
    if not folder.exists():
        write_random_model(folder, config_from_dict(dict(TOY_BLOCK)), seed=9, std=0.2,
                           norm_jitter=0.1)
    return load_model(folder, dtype, DEV)


def test_the_toy_norm_is_a_layer_norm():
    """The toy's kernel against torch: all rows with an update that joins the stream, and some
    rows only, which leaves the stream as it was."""
    lib = toy_block_library()
    g = torch.Generator().manual_seed(4)
    T, D, eps = 7, 70, 1e-3
    resid, delta = torch.randn(T, D, generator=g), torch.randn(T, D, generator=g)
    w, b = torch.randn(D, generator=g), torch.randn(D, generator=g)
    want = torch.nn.functional.layer_norm((resid + delta).double(), (D,), w.double(), b.double(), eps)

    def launch(r, d, out, rows):
        rc = lib.toy_layer_norm_launch(
            c_void_p(r.data_ptr()), c_void_p(d.data_ptr()), c_int(2), c_void_p(wd.data_ptr()),
            c_void_p(bd.data_ptr()), c_void_p(out.data_ptr()), c_int(0),
            c_void_p(rows.data_ptr() if rows is not None else 0), c_int(out.shape[0]), c_int(D),
            ctypes.c_float(eps), c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0
    wd, bd = w.to(DEV), b.to(DEV)
    r, d = resid.to(DEV), delta.to(DEV)
    out = torch.empty(T, D, device=DEV)
    launch(r, d, out, None)
    assert float((out.cpu().double() - want).abs().max()) < 1e-5
    assert torch.equal(r.cpu(), resid + delta)
    r = resid.to(DEV)
    rows = torch.tensor([5, 0, 3], dtype=torch.int32, device=DEV)
    some = torch.empty(3, D, device=DEV)
    launch(r, d, some, rows)
    assert float((some.cpu().double() - want[[5, 0, 3]]).abs().max()) < 1e-5
    assert torch.equal(r.cpu(), resid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_and_a_block_from_outside_run_from_c(tmp_path, dtype):
    """An architecture whose blocks are the toy arrangement (around the framework's conv and
    attention mixers) and the framework's own (with the toy norm as its second norm), toy norm
    before the head: launched from C it gives bit for bit what the host's part-by-part walk
    gives under the mixed schedule, with and without decode graphs, and the portions give what
    whole prompts give."""
    import schedules
    from replay_common import collect, make_requests
    model = toy_block_model(tmp_path, dtype)
    requests = make_requests(TOY_BLOCK["vocab_size"], [70, 45, 100, 37, 83, 64, 29], seed=23)
    steps, index, peak = schedules.mixed(requests)
    results = {}
    for c_forward in (True, False):
        for graphs in (False, True):
            res, runner = replay(model, steps, peak, tmp_path / f"b{c_forward}g{graphs}",
                                 c_forward, graphs)
            assert (runner._cplan is not None) == c_forward, "the toy blocks have descriptions"
            if graphs:
                assert runner.graph_replays > 0
            results[(c_forward, graphs)] = res
    base = results[(False, False)]
    for key, res in results.items():
        for a, b in zip(base, res):
            assert (a is None) == (b is None)
            if a is not None:
                assert np.array_equal(a, b), key
    whole_steps, whole_index, whole_peak = schedules.whole(requests)
    whole, _ = replay(model, whole_steps, whole_peak, tmp_path / "bwhole", True, False)
    vocab = TOY_BLOCK["vocab_size"]
    got = collect(index, {s["step"]: r for s, r in zip(steps, base) if r is not None}, vocab)
    ref = collect(whole_index, {s["step"]: r for s, r in zip(whole_steps, whole) if r is not None},
                  vocab)
    scale = max(float(np.abs(v).max()) for v in ref.values())
    tol = 2e-5 if dtype == "float32" else 4e-2
    worst = max(float(np.abs(got[k] - ref[k]).max()) for k in ref) / scale
    assert worst < tol, worst


def test_the_toy_block_does_what_it_says_inside_the_model(tmp_path):
    """A sequence through the model with the mixers and feed-forwards of all blocks but the first
    switched off (their last products zero): the logits are head(LN(x + conv(h) + ffn(h))) with
    h = LN(embedding), worked out in float64 from the file's tensors with the plain
    implementation's conv mixer and feed-forward, against the C walk."""
    from plain import lfm2 as P
    model = toy_block_model(tmp_path, "float32")
    for blk in model.layers[1:]:
        blk.feed_forward.down.weight.zero_()
        mixer_out = blk.mixer.out if hasattr(blk.mixer, "out") else blk.mixer.out_proj
        mixer_out.weight.zero_()
        if mixer_out.bias is not None:
            mixer_out.bias.zero_()
    toks = [int(t) for t in np.random.default_rng(5).integers(0, TOY_BLOCK["vocab_size"], size=11)]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks, "want": list(range(11))}],
              "end": ["a"]}]
    (got,), runner = replay(model, steps, 64, tmp_path / "bzero", True, False)
    assert runner._cplan is not None
    w = {k: np.asarray(v, dtype=np.float64) for k, v in
         P.read_safetensors(tmp_path / "toy_block" / "model.safetensors").items()}

    def ln(x, name):
        mu = x.mean(-1, keepdims=True)
        var = ((x - mu) ** 2).mean(-1, keepdims=True)
        return (x - mu) / np.sqrt(var + TOY_BLOCK["eps"]) * w[name + ".weight"] + w[name + ".bias"]
    x = w["emb.weight"][toks]
    h = ln(x, "blocks.0.n")
    conv = {"in_proj": w["blocks.0.conv.in_proj.weight"], "in_proj_bias": w["blocks.0.conv.in_proj.bias"],
            "conv": w["blocks.0.conv.conv.weight"].reshape(TOY_BLOCK["width"], TOY_BLOCK["taps"]),
            "conv_bias": w["blocks.0.conv.conv.bias"], "out_proj": w["blocks.0.conv.out_proj.weight"],
            "out_proj_bias": w["blocks.0.conv.out_proj.bias"]}
    ff = {k: w[f"blocks.0.ff.{k}.weight"] for k in ("w1", "w2", "w3")}
    x = x + P.short_conv_mixer(h, conv, {"hidden_size": TOY_BLOCK["width"]}) + P.swiglu_feed_forward(h, ff)
    want = ln(x, "final") @ w["emb.weight"].T
    assert float(np.abs(got - want).max()) < 2e-5 * float(np.abs(want).max())


# ---------------------------------------------------------------------------------------------
# an encoding of positions from outside, added to the embedded rows
# ---------------------------------------------------------------------------------------------
def toy_positions_library():
    from kappai_amd.kernels.lib import library_at
    lib = library_at(TOY_POSITIONS_SOURCE)
    lib.toy_learned_positions_run.restype = None
    return lib


def define_toy_positions():
    from kappai_amd.config import ModelConfig, register_architecture
    from kappai_amd.kernels import ops
    from kappai_amd.models import Model
    from kappai_amd.parts import (POSITION_ENCODINGS, OutputHead, PositionEncoding,
                                  TokenEmbedding, make_part, register_part)
    from kappai_amd.parts.base import StepTables
    from kappai_amd.parts.cdesc import RUNNER_EMBEDDED
    from kappai_amd.weights.spec import INIT_NORMAL, TABLE, TensorSpec
    if "toy_learned_hip" in POSITION_ENCODINGS:
        return

    class PositionsDesc(Structure):
        """``toy_learned_positions`` of tests/toy_parts/learned_positions.hip."""
        _fields_ = [("table", c_void_p), ("table_is_bf16", c_int), ("positions", c_int),
                    ("rows_table", c_int)]

    class TableRows(StepTables):
        """A table of the step that the part lays out itself, on the host: the table's row for
        every row of the step (its position, the last row for anything beyond).  It depends on the
        positions, so a captured decode graph has it built again for every replay."""
        family = "toy_table_rows"
        decode_constant = False

        def __init__(self, n):
            self.n = n

        def __eq__(self, other):
            return isinstance(other, TableRows) and other.n == self.n

        def build(self, step):
            TableRows.built += 1
            return {"toy_table_rows": np.minimum(step.arrays["row_pos"], self.n - 1).astype(np.int32)}, {}

    TableRows.built = 0

    class LearnedPositionsHip(PositionEncoding):
        """x_t += table[position of t]."""

        def __init__(self, name, n_positions, width):
            self.name, self.n, self.width = name, n_positions, width
            self.step_tables = TableRows(n_positions)

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.n, self.width), TABLE, INIT_NORMAL)]

        def bind(self, tensors):
            self.table = tensors[self.name + ".weight"].contiguous()

        def on_embedding(self, x, batch):
            rc = toy_positions_library().toy_add_positions_launch(
                c_void_p(x.data_ptr()), c_void_p(self.table.data_ptr()),
                c_int(1 if self.table.dtype == torch.bfloat16 else 0),
                c_void_p(batch.extra["toy_table_rows"].data_ptr()), c_int(x.shape[0]),
                c_int(self.width), c_int(self.n), ops._stream())
            assert rc == 0, rc

        def c_embedded(self, plan):
            lib = toy_positions_library()
            assert lib.toy_learned_positions_desc_bytes() == ctypes.sizeof(PositionsDesc)
            plan.register_runner("embedded.toy_learned", RUNNER_EMBEDDED,
                                 lib.toy_learned_positions_run, PositionsDesc)
            return plan.embedded("embedded.toy_learned", PositionsDesc(
                self.table.data_ptr(), 1 if self.table.dtype == torch.bfloat16 else 0, self.n,
                plan.table("toy_table_rows")))

    register_part("position_encoding", "toy_learned_hip", LearnedPositionsHip)

    @dataclass
    class ToyPositionsConfig(ModelConfig):
        width: int = 0
        vocab_size: int = 0
        heads: int = 0
        head_dim: int = 0
        ff: int = 0
        eps: float = 1e-5
        max_position_embeddings: int = 256

        KEYS = ("width", "vocab_size", "heads", "head_dim", "ff", "eps")

        @classmethod
        def from_dict(cls, raw):
            return cls(architecture="ToyPositionsForCausalLM", **{k: raw[k] for k in cls.KEYS})

        def to_dict(self):
            return {"architectures": ["ToyPositionsForCausalLM"],
                    **{k: getattr(self, k) for k in self.KEYS}}

    def build(cfg, dtype):
        def rms(name):
            return make_part("norm", "rmsnorm", name=name, width=cfg.width, eps=cfg.eps,
                             dtype=dtype)

        def block(i, mixer):
            p = f"blocks.{i}."
            return make_part("block", "pre_norm", mixer_norm=rms(p + "n1"), mixer=mixer,
                             ffn_norm=rms(p + "n2"),
                             feed_forward=make_part("feed_forward", "swiglu", prefix=p + "ff.",
                                                    width=cfg.width, hidden=cfg.ff, dtype=dtype))
        # attention without rotation: the positions come from the table alone
        layers = [block(i, make_part("mixer", "attention", prefix=f"blocks.{i}.att.",
                                     width=cfg.width, num_heads=cfg.heads,
                                     num_kv_heads=cfg.heads // 2, head_dim=cfg.head_dim,
                                     dtype=dtype, position=None, qk_norm_eps=None))
                  for i in range(2)]
        emb = TokenEmbedding("emb", cfg.vocab_size, cfg.width)
        positions = make_part("position_encoding", "toy_learned_hip", name="pos",
                              n_positions=cfg.max_position_embeddings, width=cfg.width)
        return Model(cfg, dtype, emb, layers, rms("final"),
                     OutputHead("head", cfg.vocab_size, cfg.width, tied_to=emb),
                     embedding_position=positions)

    register_architecture("ToyPositionsForCausalLM", ToyPositionsConfig, build)


TOY_POSITIONS = {"architectures": ["ToyPositionsForCausalLM"], "width": 64, "vocab_size": 131,
                 "heads": 4, "head_dim": 16, "ff": 96, "eps": 1e-5}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_positions_added_to_the_embedded_rows_run_from_c(tmp_path, dtype):
    """A learned row per position added to the embedded rows by a kernel from outside, attention
    without rotation, the kernel reading a table of the step that the part lays out itself
    (``StepTables``, beside the attention's tiles; built again for every replay of a decode
    graph): from C bit for bit what the host's walk gives under the mixed schedule, with and
    without graphs; and the model does depend on the positions (a request whose table rows are
    moved gives other logits)."""
    import schedules
    from kappai_amd.config import config_from_dict
    from kappai_amd.models import load_model
    from kappai_amd.weights import write_random_model
    from replay_common import make_requests
    define_toy_positions()
    folder = tmp_path / "toy_positions"
    write_random_model(folder, config_from_dict(dict(TOY_POSITIONS)), seed=11, std=0.2,
                       norm_jitter=0.1)
    model = load_model(folder, dtype, DEV)
    requests = make_requests(TOY_POSITIONS["vocab_size"], [70, 45, 100, 37, 83], seed=24)
    steps, index, peak = schedules.mixed(requests)
    results = {}
    for c_forward in (True, False):
        for graphs in (False, True):
            res, runner = replay(model, steps, peak, tmp_path / f"p{c_forward}g{graphs}",
                                 c_forward, graphs)
            assert (runner._cplan is not None) == c_forward
            assert sorted(t.family for t in runner.step_tables) == ["attention_tiles",
                                                                    "toy_table_rows"]
            if graphs:
                assert runner.graph_replays > 0
            results[(c_forward, graphs)] = res
    base = results[(False, False)]
    for key, res in results.items():
        for a, b in zip(base, res):
            assert (a is None) == (b is None)
            if a is not None:
                assert np.array_equal(a, b), key
    # the positions matter: with the table's rows rolled by one the logits move
    model.embedding_position.table.copy_(torch.roll(model.embedding_position.table, 1, 0))
    moved, _ = replay(model, steps, peak, tmp_path / "pmoved", True, False)
    first = next(i for i, a in enumerate(base) if a is not None)
    assert float(np.abs(moved[first] - base[first]).max()) > 1e-3
