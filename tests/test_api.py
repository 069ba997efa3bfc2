"""The drop-in Python API: compress_model -> DF11 safetensors -> DFloat11Model.from_pretrained,
with the reference's names, files and error behaviour (no GPU needed for these)."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn as nn
from safetensors.torch import load_file

from dfloat11_amd import DFloat11Model, compress_model
from dfloat11_amd import dfloat11 as M


class Block(nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.attn = nn.Module()
        self.attn.q_proj = nn.Linear(d, d, bias=False)
        self.attn.o_proj = nn.Linear(d, d, bias=True)
        self.mlp = nn.Module()
        self.mlp.up = nn.Linear(d, h, bias=False)
        self.mlp.down = nn.Linear(h, d, bias=False)
        self.norm = nn.LayerNorm(d)

    def forward(self, x):
        x = x + self.attn.o_proj(self.attn.q_proj(self.norm(x)))
        return x + self.mlp.down(torch.relu(self.mlp.up(x)))


class Tiny(nn.Module):
    def __init__(self, vocab=97, d=64, h=160, n_layers=3):
        super().__init__()
        self.embed = nn.Embedding(vocab, d)
        self.layers = nn.ModuleList([Block(d, h) for _ in range(n_layers)])
        self.lm_head = nn.Linear(d, vocab, bias=False)

    def forward(self, ids):
        x = self.embed(ids)
        for layer in self.layers:
            x = layer(x)
        return self.lm_head(x)


PATTERNS = {
    r"embed": [],
    r"layers\.\d+": ["attn.q_proj", "attn.o_proj", "mlp.up", "mlp.down"],
    r"lm_head": [],
}


def make_model(seed=0):
    torch.manual_seed(seed)
    m = Tiny().to(torch.bfloat16)
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() > 1:
                p.copy_((torch.randn(p.shape) * 0.02).to(torch.bfloat16))
    return m.eval()


@pytest.fixture()
def compressed(tmp_path):
    model = make_model()
    originals = {k: v.clone() for k, v in model.state_dict().items()}
    compress_model(model, PATTERNS, str(tmp_path), check_correctness=False)
    return tmp_path, originals


def test_files_and_config(compressed):
    path, originals = compressed
    assert sorted(os.listdir(path)) == ["config.json", "model.safetensors"]
    cfg = json.load(open(path / "config.json"))["dfloat11_config"]
    assert cfg == {"version": "0.5.0", "threads_per_block": [512], "bytes_per_thread": 8,
                   "pattern_dict": PATTERNS}
    tensors = load_file(str(path / "model.safetensors"))
    for mod in ("embed", "layers.0", "layers.2", "lm_head"):
        for name, dtype in (("luts", torch.uint8), ("encoded_exponent", torch.uint8),
                            ("sign_mantissa", torch.uint8), ("output_positions", torch.uint8),
                            ("gaps", torch.uint8), ("split_positions", torch.int64)):
            assert tensors[f"{mod}.{name}"].dtype == dtype
    assert "layers.0.attn.q_proj.weight" not in tensors and "embed.weight" not in tensors
    assert "layers.0.attn.o_proj.bias" in tensors and "layers.1.norm.weight" in tensors
    # a block stores its four weights as ONE stream, split points between them
    assert tensors["layers.1.split_positions"].tolist() == [64 * 64, 2 * 64 * 64, 2 * 64 * 64 + 160 * 64]
    assert tensors["embed.split_positions"].numel() == 0
    n = 2 * 64 * 64 + 2 * 160 * 64
    assert tensors["layers.1.sign_mantissa"].numel() == n
    n_blocks = -(-tensors["layers.1.encoded_exponent"].numel() // 4096)
    assert tensors["layers.1.gaps"].numel() == 320 * n_blocks
    assert tensors["layers.1.output_positions"].numel() == 4 * (n_blocks + 1)
    assert tensors["layers.1.luts"].shape[1] == 256


def test_streams_decode_to_the_original_weights(compressed, oracle):
    """What compress_model wrote, read back with the oracle's restatement of the reference kernel."""
    path, originals = compressed
    t = load_file(str(path / "model.safetensors"))
    for mod, names in (("embed", ["embed.weight"]), ("lm_head", ["lm_head.weight"]),
                       ("layers.2", [f"layers.2.{a}.weight" for a in PATTERNS[r"layers\.\d+"]])):
        out = oracle.c_decode(t[f"{mod}.luts"].numpy(), t[f"{mod}.encoded_exponent"].numpy(),
                              t[f"{mod}.sign_mantissa"].numpy(), t[f"{mod}.output_positions"].numpy(),
                              t[f"{mod}.gaps"].numpy())
        want = torch.cat([originals[n].flatten() for n in names]).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(out, want)


def test_loader_installs_hooks_and_drops_weights(compressed):
    path, originals = compressed
    model = DFloat11Model.from_pretrained(str(path), device="cpu", bfloat16_model=make_model(seed=1))
    for mod in (model.embed, model.layers[0], model.lm_head):
        assert len(mod._forward_pre_hooks) == 1
        assert mod.luts.dtype == torch.uint8 and mod.output_positions.dtype == torch.uint8
        assert isinstance(mod.shared_mem_size, int) and mod.shared_mem_size > 2052
    assert not hasattr(model.embed, "weight") and not hasattr(model.lm_head, "weight")
    blk = model.layers[1]
    assert [type(m) for m in blk.weight_injection_modules] == [nn.Linear] * 4
    assert not hasattr(blk.attn.q_proj, "weight") and not hasattr(blk.mlp.down, "weight")
    assert isinstance(blk.split_positions, list) and len(blk.split_positions) == 3
    # uncompressed tensors were copied into the fresh model
    assert torch.equal(model.layers[0].attn.o_proj.bias, originals["layers.0.attn.o_proj.bias"])
    assert torch.equal(model.layers[2].norm.weight, originals["layers.2.norm.weight"])


def test_forward_on_cpu_fails_loudly(compressed):
    path, _ = compressed
    model = DFloat11Model.from_pretrained(str(path), device="cpu", bfloat16_model=make_model(seed=1))
    with pytest.raises(RuntimeError, match="GPU"):
        model(torch.zeros(1, 4, dtype=torch.long))


def test_cpu_offload_keeps_streams_on_the_host(compressed):
    path, _ = compressed
    model = DFloat11Model.from_pretrained(str(path), device="cpu", bfloat16_model=make_model(seed=1),
                                          cpu_offload=True, cpu_offload_blocks=2, pin_memory=False)
    offloaded = [m for m in (model.embed, *model.layers, model.lm_head) if hasattr(m, "offloaded_tensors")]
    assert len(offloaded) == 2
    for m in offloaded:
        assert set(m.offloaded_tensors) == {"encoded_exponent", "sign_mantissa"}
        assert not hasattr(m, "encoded_exponent") and hasattr(m, "luts") and hasattr(m, "gaps")


def test_single_file_and_error_paths(compressed, tmp_path):
    path, _ = compressed
    f = str(path / "model.safetensors")
    model = DFloat11Model.from_single_file(f, pattern_dict=PATTERNS, bfloat16_model=make_model(seed=2), device="cpu")
    assert hasattr(model.embed, "luts")
    with pytest.raises(IsADirectoryError):
        DFloat11Model.from_single_file(str(path), pattern_dict=PATTERNS, bfloat16_model=make_model(), device="cpu")
    with pytest.raises(FileNotFoundError):
        DFloat11Model.from_single_file(str(path / "nope.safetensors"), pattern_dict=PATTERNS,
                                       bfloat16_model=make_model(), device="cpu")
    # a directory whose config.json lacks dfloat11_config
    bad = tmp_path / "bad"
    bad.mkdir()
    (bad / "config.json").write_text("{}")
    with pytest.raises(AttributeError, match="dfloat11_config"):
        DFloat11Model.from_pretrained(str(bad), device="cpu", bfloat16_model=make_model())


def test_block_range_and_sharded_save(tmp_path):
    model = make_model()
    compress_model(model, PATTERNS, str(tmp_path), block_range=[1, 3], save_single_file=False,
                   check_correctness=False)
    files = sorted(os.listdir(tmp_path))
    # blocks 2 and 3 of the walk (layers.0, layers.1) are written; the walk stops at block 4, so
    # neither the rest of the model nor config.json is saved by this invocation
    assert files == ["layers_0.safetensors", "layers_1.safetensors"]
    t = load_file(str(tmp_path / "layers_1.safetensors"))
    assert "layers.1.encoded_exponent" in t and "layers.1.attn.o_proj.bias" in t


def test_non_bf16_weights_are_rejected(tmp_path):
    model = make_model().float()
    with pytest.raises(AssertionError, match="bfloat16"):
        compress_model(model, PATTERNS, str(tmp_path), check_correctness=False)


def test_check_correctness_needs_a_gpu(tmp_path):
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError, match="GPU"):
        compress_model(make_model(), PATTERNS, str(tmp_path), check_correctness=True)


def test_tensor_manager_is_grow_only():
    M.TensorManager.clear()
    a = M.TensorManager.allocate_bfloat16("cpu", 100)
    b = M.TensorManager.allocate_bfloat16(torch.device("cpu"), 40)
    assert a.numel() == 100 and b.numel() == 40 and b.data_ptr() == a.data_ptr()
    c = M.TensorManager.allocate_bfloat16("cpu", 1000)
    assert c.numel() == 1000
    M.TensorManager.clear()


def test_unsupported_stream_geometry_is_rejected():
    with pytest.raises(NotImplementedError):
        M.get_hook((256, ), 8)


def test_validate_stream_accepts_good_and_names_what_is_wrong():
    """Load-time layout check (the reference has none: a malformed stream makes its
    kernel read or write out of bounds)."""
    import numpy as np
    from dfloat11_amd import decode as D
    from dfloat11_amd._native import DF11Error
    from tests.df11_cases import compress_product, make_case
    c = compress_product(make_case("normal", 30_000, 5))
    t = {k: torch.from_numpy(np.ascontiguousarray(c[k])) for k in
         ("luts", "encoded_exponent", "sign_mantissa", "gaps")}
    pos = torch.from_numpy(np.ascontiguousarray(c["output_positions"]).view(np.uint8).copy())

    def check(**over):
        a = dict(t, output_positions=pos)
        a.update(over)
        D.validate_stream(a["luts"], a["encoded_exponent"], a["sign_mantissa"], a["output_positions"], a["gaps"])

    check()
    check(output_positions=pos[:-4])                      # the reference's own files may lack the final entry
    bad_pos = pos.clone().view(torch.int32)
    bad_pos[1] = bad_pos[2] + 1
    for over, word in ((dict(gaps=t["gaps"][:-1]), "gaps"),
                       (dict(output_positions=bad_pos.view(torch.uint8)), "decrease"),
                       (dict(sign_mantissa=t["sign_mantissa"][:-1]), "last position"),
                       (dict(luts=t["luts"][:1]), "luts"),
                       (dict(output_positions=pos[:-8]), "entries")):
        with pytest.raises(DF11Error, match=word):
            check(**over)


def test_compress_cli_on_a_local_checkpoint(tmp_path):
    """python -m dfloat11_amd.compress: a saved transformers checkpoint in, a DF11
    directory with config and per-block safetensors out, streams decode to the weights."""
    import json
    from safetensors.torch import load_file
    from transformers import AutoModelForCausalLM, LlamaConfig
    from dfloat11_amd import compress
    cfg = LlamaConfig(vocab_size=300, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=64,
                      tie_word_embeddings=True)
    torch.manual_seed(0)
    src, dst = tmp_path / "bf16", tmp_path / "df11"
    base = AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16)
    base.save_pretrained(str(src))
    compress.main(["--model_name_or_path", str(src), "--save_path", str(dst)])
    conf = json.load(open(dst / "config.json"))
    assert conf["dfloat11_config"]["bytes_per_thread"] == 8 and conf["tie_word_embeddings"] is False
    files = sorted(p.name for p in dst.glob("*.safetensors"))
    assert "model_layers_0.safetensors" in files and "lm_head.safetensors" in files
    layer = load_file(str(dst / "model_layers_1.safetensors"))
    assert {"model.layers.1.luts", "model.layers.1.encoded_exponent", "model.layers.1.sign_mantissa",
            "model.layers.1.output_positions", "model.layers.1.gaps",
            "model.layers.1.split_positions"} <= set(layer)
    want = torch.cat([base.get_submodule(f"model.layers.1.{n}").weight.detach().flatten()
                      for n in compress.LLM_PATTERNS[r"model\.layers\.\d+"]])
    assert layer["model.layers.1.sign_mantissa"].numel() == want.numel()


class _StubPrefetcher(M._OffloadPrefetcher):
    """The prefetcher's bookkeeping without a GPU: copies, waits and events are recorded, not run."""

    def __init__(self):
        super().__init__()
        self.log = []

    def _copy_to_slots(self, module, device, parity):
        self.log.append(("copy", module.name, parity))
        tensors = {name: self._slot(device, parity, name, host) for name, host in module.offloaded_tensors.items()}
        for name, dst in tensors.items():
            dst.copy_(module.offloaded_tensors[name])
        return tensors, object()

    def _wait_and_mark(self, device, tensors, done):
        pass

    def _decode_done_event(self, device):
        return object()


class _Offloaded(nn.Module):
    def __init__(self, name, n):
        super().__init__()
        self.name = name
        self.offloaded_tensors = {"encoded_exponent": torch.full((n,), len(name), dtype=torch.uint8),
                                  "sign_mantissa": torch.arange(n, dtype=torch.uint8)}


def test_prefetcher_learns_the_order_and_lets_go_of_dead_modules():
    import gc
    import weakref
    p = _StubPrefetcher()
    dev = torch.device("cpu")          # stands in for a GPU: the stub never touches it
    mods = [_Offloaded(f"m{i}", 10 + i) for i in range(3)]

    def forward(order):
        for m in order:
            tensors, parity = p.fetch(m, dev)
            assert torch.equal(tensors["sign_mantissa"], m.offloaded_tensors["sign_mantissa"])
            assert torch.equal(tensors["encoded_exponent"], m.offloaded_tensors["encoded_exponent"])
            p.after_decode(m, dev, parity)

    forward(mods)                      # first pass: every copy is issued by the module itself
    assert [e[1] for e in p.log] == ["m0", "m1", "m2"]
    assert [e[2] for e in p.log] == [0, 1, 0]          # the two slots alternate
    p.log.clear()
    forward(mods)                      # second pass: m0 copies itself, the others were copied one module ahead
    assert [e[1] for e in p.log] == ["m0", "m1", "m2", "m0"]
    p.log.clear()
    forward([mods[0], mods[2]])        # a block skipped: the copy made for m1 is dropped, m2 fetches its own
    assert [e[1] for e in p.log] == ["m1", "m2", "m0"] and not p._prefetched(mods[1], dev)
    forward(mods)
    # deleting the modules releases everything that was kept for them, without reset()
    refs = [weakref.ref(m) for m in mods]
    assert p.live == {dev: 3} and p.slots
    del mods
    gc.collect()
    assert all(r() is None for r in refs)
    assert not p.live and not p.slots and not p.slot_owner and not p.slot_free and not p.last
    assert len(p.pending) == 0 and len(p.successor) == 0


def test_prefetcher_reset_voids_earlier_finalizers():
    import gc
    p = _StubPrefetcher()
    dev = torch.device("cpu")
    old = _Offloaded("old", 4)
    p.fetch(old, dev)
    p.reset()
    p.log = []
    new = _Offloaded("new", 4)
    tensors, parity = p.fetch(new, dev)
    del old
    gc.collect()
    assert p.live == {dev: 1} and p.slots      # the death of a module from before the reset changes nothing


def test_hook_takes_each_stream_from_where_it_is(monkeypatch):
    """A module with only one of its two large streams offloaded (tensor names of different
    modules interleave in a file and cpu_offload_blocks runs out in between): the hook
    takes that stream from the prefetcher and the other from the module's buffer."""
    calls = {}
    mod = nn.Linear(4, 2, bias=False).to(torch.bfloat16)
    delattr(mod, "weight")
    mod.register_buffer("luts", torch.zeros(2, 256, dtype=torch.uint8))
    mod.register_buffer("sign_mantissa", torch.arange(8, dtype=torch.uint8))
    mod.register_buffer("output_positions", torch.zeros(8, dtype=torch.uint8))
    mod.register_buffer("gaps", torch.zeros(320, dtype=torch.uint8))
    mod.offloaded_tensors = {"encoded_exponent": torch.ones(16, dtype=torch.uint8)}
    mod.split_positions = []
    staged = torch.full((16,), 7, dtype=torch.uint8)

    class FakeDevice:
        type = "cuda"
    monkeypatch.setattr(type(mod.luts), "device", property(lambda self: FakeDevice()), raising=False)
    monkeypatch.setattr(M._prefetcher, "fetch", lambda module, device: ({"encoded_exponent": staged}, 1))
    monkeypatch.setattr(M._prefetcher, "after_decode", lambda module, device, parity: calls.setdefault("after", parity))
    monkeypatch.setattr(M.TensorManager, "allocate_bfloat16",
                        staticmethod(lambda device, n: torch.zeros(n, dtype=torch.bfloat16)))
    monkeypatch.setattr(M._decode, "validate_stream", lambda *a, **k: None)
    monkeypatch.setattr(M._decode, "prepare", lambda *a, **k: (torch.zeros(16, dtype=torch.uint8), 5))

    def bind(luts, enc, sm, pos, gaps, out, ws, max_sub):
        calls["bind"] = (enc, sm)
        return ()
    monkeypatch.setattr(M._decode, "bind", bind)
    monkeypatch.setattr(M._decode, "launch", lambda bound, device: calls.setdefault("launched", True))
    M.get_hook((512,), 8)(mod, None)
    assert calls["bind"][0] is staged and calls["bind"][1] is mod.sign_mantissa
    assert calls["launched"] and calls["after"] == 1 and mod.weight.shape == (2, 4)
