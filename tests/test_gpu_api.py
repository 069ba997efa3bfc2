"""The drop-in API on a real MI355X: a DF11 model's outputs are bit-identical to the BF16 model's."""
import pytest
import torch

from dfloat11_amd import DFloat11Model, compress_model
from dfloat11_amd import dfloat11 as M
from tests.test_api import PATTERNS, make_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _reference_logits(seed, ids):
    ref = make_model(seed).to(DEV)
    with torch.no_grad():
        return ref(ids)


@pytest.mark.parametrize("offload", [False, True])
def test_forward_bit_identical(tmp_path, offload):
    print(f"case api forward offload={offload}", flush=True)
    M._prefetcher.reset()
    compress_model(make_model(3), PATTERNS, str(tmp_path), check_correctness=True, check_device=DEV)
    model = DFloat11Model.from_pretrained(str(tmp_path), device=DEV, bfloat16_model=make_model(9),
                                          cpu_offload=offload)
    ids = torch.randint(0, 97, (4, 16), device=DEV)
    want = _reference_logits(3, ids)
    with torch.no_grad():
        for _ in range(3):                       # later passes run with the prefetch order learnt
            got = model(ids)
            assert torch.equal(got, want)
    # derived workspaces are attributes, not part of the saved state
    assert not any("_df11" in k for k in model.state_dict())
    if offload:
        assert not hasattr(model.layers[0], "encoded_exponent")
        assert model.layers[0].offloaded_tensors["encoded_exponent"].is_pinned()


def test_offload_prefetch_survives_a_changing_module_order(tmp_path):
    """Blocks skipped, run in reverse or twice: the prefetcher's guess of the next
    module is then wrong, and a staging slot it filled for one module is handed to
    another before the first ever runs.  Every pass must still decode each
    module's own streams."""
    print("case api offload, changing order", flush=True)
    M._prefetcher.reset()
    compress_model(make_model(5), PATTERNS, str(tmp_path), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path), device=DEV, bfloat16_model=make_model(9),
                                          cpu_offload=True)
    ref = make_model(5).to(DEV)
    ids = torch.randint(0, 97, (2, 8), device=DEV)

    def run(m, order):
        x = m.embed(ids)
        for i in order:
            x = m.layers[i](x)
        return m.lm_head(x)

    with torch.no_grad():
        for order in ([0, 1, 2], [0, 2], [0, 1, 2], [2], [0, 1, 2], [2, 1, 0], [1, 1, 0], [0, 1, 2], [], [0, 1, 2]):
            assert torch.equal(run(model, order), run(ref, order)), order


def test_model_moved_between_cpu_and_gpu(tmp_path):
    """Loaded on the CPU and moved later, moved away and back (what accelerate's
    model offload does around every forward): the streams follow the module, the
    decode binds to the tensors that are there now."""
    print("case api cpu <-> gpu moves", flush=True)
    M._prefetcher.reset()
    compress_model(make_model(6), PATTERNS, str(tmp_path), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path), device="cpu", bfloat16_model=make_model(9))
    ids = torch.randint(0, 97, (2, 8), device=DEV)
    want = _reference_logits(6, ids)
    with pytest.raises(RuntimeError):
        model(ids.cpu())                      # no CPU decode path
    with torch.no_grad():
        model = model.to(DEV)
        assert torch.equal(model(ids), want)
        assert torch.equal(model(ids), want)
        model = model.to("cpu")
        model = model.to(DEV)
        assert torch.equal(model(ids), want)
        assert torch.equal(model(ids), want)


def test_replaced_weight_attribute_is_reinjected(tmp_path):
    """As in the reference, every forward puts the decoded weights back in place
    (dfloat11.py:153-166), also after someone assigned another tensor to `weight`."""
    print("case api weight replaced", flush=True)
    M._prefetcher.reset()
    compress_model(make_model(7), PATTERNS, str(tmp_path), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path), device=DEV, bfloat16_model=make_model(9))
    ids = torch.randint(0, 97, (2, 8), device=DEV)
    want = _reference_logits(7, ids)
    with torch.no_grad():
        assert torch.equal(model(ids), want)
        assert torch.equal(model(ids), want)          # second call: launch arguments already bound
        lin = model.layers[1].mlp.up
        lin.weight = torch.zeros_like(lin.weight)
        model.lm_head.weight = torch.ones_like(model.lm_head.weight)
        assert torch.equal(model(ids), want)
        assert torch.equal(model(ids), want)


def test_shared_buffer_is_reused_across_modules(tmp_path):
    print("case api shared buffer", flush=True)
    M.TensorManager.clear()
    compress_model(make_model(4), PATTERNS, str(tmp_path), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path), device=DEV, bfloat16_model=make_model(9))
    ids = torch.randint(0, 97, (2, 8), device=DEV)
    with torch.no_grad():
        model(ids)
    buf = M.TensorManager._tensors[torch.device(DEV)]
    biggest = max(2 * 64 * 64 + 2 * 160 * 64, 97 * 64)
    assert buf.numel() == biggest
    # every injected weight is a view into that one buffer
    for lin in model.layers[2].weight_injection_modules:
        assert buf.data_ptr() <= lin.weight.data_ptr() < buf.data_ptr() + buf.numel() * 2


def test_hf_llama_generate_matches_bf16(tmp_path):
    """transformers path: save_pretrained + AutoConfig, greedy generation token-identical."""
    print("case api hf llama", flush=True)
    from transformers import AutoModelForCausalLM, LlamaConfig
    cfg = LlamaConfig(vocab_size=512, hidden_size=128, intermediate_size=256, num_hidden_layers=3,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128,
                      tie_word_embeddings=False)
    torch.manual_seed(0)
    base = AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16).eval()
    ref = AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16).eval()
    ref.load_state_dict(base.state_dict())
    patterns = {r"model\.embed_tokens": [], r"lm_head": [],
                r"model\.layers\.\d+": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj",
                                        "self_attn.o_proj", "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"]}
    compress_model(base, patterns, str(tmp_path), save_single_file=False, check_correctness=True,
                   check_device=DEV)
    model = DFloat11Model.from_pretrained(str(tmp_path), device=DEV)
    ref = ref.to(DEV)
    ids = torch.randint(0, 512, (2, 12), device=DEV)
    with torch.no_grad():
        assert torch.equal(model(ids).logits, ref(ids).logits)
        a = model.generate(ids, max_new_tokens=16, do_sample=False)
        b = ref.generate(ids, max_new_tokens=16, do_sample=False)
    assert torch.equal(a, b)


def test_hf_llama_device_map_auto(tmp_path):
    """The reference's default call: no device given, device_map='auto' (accelerate
    places whole compressed blocks; with one GPU everything lands on it)."""
    print("case api device_map auto", flush=True)
    from transformers import AutoModelForCausalLM, LlamaConfig
    cfg = LlamaConfig(vocab_size=384, hidden_size=64, intermediate_size=192, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=64,
                      tie_word_embeddings=False)
    torch.manual_seed(1)
    base = AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16).eval()
    ref = AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16).eval()
    ref.load_state_dict(base.state_dict())
    patterns = {r"model\.embed_tokens": [], r"lm_head": [],
                r"model\.layers\.\d+": ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj",
                                        "self_attn.o_proj", "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"]}
    compress_model(base, patterns, str(tmp_path), save_single_file=False, check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path))
    assert all(b.device.type == "cuda" for b in model.buffers())
    ref = ref.to(DEV)
    ids = torch.randint(0, 384, (2, 9), device=DEV)
    with torch.no_grad():
        assert torch.equal(model(ids).logits, ref(ids).logits)


def test_inference_cli_synthetic_matches_bf16():
    """The generation benchmark on a small random-init Qwen3-shaped model with tied
    embeddings: DF11 logits and greedy tokens are bit-identical to BF16's."""
    print("case api inference cli", flush=True)
    from dfloat11_amd import inference
    M._prefetcher.reset()
    report = inference.main(["--synthetic", "tiny", "--num_tokens", "12", "--batch_size", "3",
                             "--prompt_len", "9", "--compare_bf16", "--json", "--device", DEV])
    assert report["logits_bit_identical"] and report["tokens_identical"]
    assert report["df11"]["new_tokens_per_sequence"] == 12
    assert 0.5 < report["compressed_over_bf16"] < 0.8


def test_compress_cli_output_loads_and_matches(tmp_path):
    """A tied-embedding checkpoint through `python -m dfloat11_amd.compress`, loaded with
    DFloat11Model.from_pretrained: logits bit-identical to the BF16 checkpoint's."""
    print("case api compress cli", flush=True)
    from transformers import AutoModelForCausalLM, LlamaConfig
    from dfloat11_amd import compress
    M._prefetcher.reset()
    cfg = LlamaConfig(vocab_size=300, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=64,
                      tie_word_embeddings=True)
    torch.manual_seed(1)
    src, dst = tmp_path / "bf16", tmp_path / "df11"
    AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16).save_pretrained(str(src))
    compress.main(["--model_name_or_path", str(src), "--save_path", str(dst), "--check_correctness"])
    ref = AutoModelForCausalLM.from_pretrained(str(src), torch_dtype=torch.bfloat16).to(DEV).eval()
    model = DFloat11Model.from_pretrained(str(dst), device=DEV)
    ids = torch.randint(0, 300, (2, 11), device=DEV)
    with torch.no_grad():
        assert torch.equal(model(ids).logits, ref(ids).logits)


def test_qwen3_8b_shape_generate_matches_bf16():
    """The full Qwen3-8B shape (36 layers, hidden 4096, MLP 12288, vocabulary 151936, tied
    embeddings; 7.57 B parameters, random-init N(0, 0.02)): prompt logits and greedy tokens
    of the DF11 model are bit-identical to the BF16 model's, at batch 1 and batch 64
    (what the reference checks per block at compression time, dfloat11.py:560-591, here
    end to end through the hooks)."""
    print("case api qwen3-8b full shape", flush=True)
    from dfloat11_amd import inference
    M._prefetcher.reset()
    M.TensorManager.clear()
    dev = torch.device(DEV)
    model = inference.build_synthetic("qwen3-8b", dev, seed=42)
    assert sum(p.numel() for p in model.parameters()) == 7_568_405_504
    batches = {}
    for batch in (1, 64):
        gen = torch.Generator(device="cpu").manual_seed(42 + batch)
        ids = torch.randint(0, model.config.vocab_size, (batch, 64), generator=gen).to(dev)
        inputs = {"input_ids": ids, "attention_mask": torch.ones_like(ids)}
        with torch.no_grad():
            logits = model(**inputs, use_cache=False).logits
            tokens = model.generate(**inputs, max_new_tokens=8, min_new_tokens=8, do_sample=False)
        batches[batch] = (inputs, logits, tokens)
    print("case api qwen3-8b full shape: compressing", flush=True)
    compressed, original = inference.convert_in_memory(model, inference.LLM_PATTERNS, dev)
    assert 0.6 < compressed / original < 0.75
    torch.cuda.empty_cache()
    assert not any(name.endswith("proj.weight") for name, _ in model.named_parameters())
    for batch, (inputs, logits, tokens) in batches.items():
        print(f"case api qwen3-8b full shape: DF11 batch {batch}", flush=True)
        with torch.no_grad():
            got_logits = model(**inputs, use_cache=False).logits
            got_tokens = model.generate(**inputs, max_new_tokens=8, min_new_tokens=8, do_sample=False)
        assert torch.equal(got_logits, logits), batch
        assert torch.equal(got_tokens, tokens), batch
    del model, batches
    M.TensorManager.clear()
    torch.cuda.empty_cache()


def test_flux_shaped_offloaded_pass_is_bit_identical():
    """FLUX.1-dev block shapes (hidden 3072, 24 heads, MLP ratio 4; module names and the
    order of the linears as in the reference's FLUX pattern_dict,
    examples/compress_flux1/compress_flux.py:49-74), two double-stream and three
    single-stream blocks, 4096 image + 512 text tokens: the pass with the compressed
    streams in pinned host memory, copied one block ahead, gives the same bits as the
    pass with resident streams and as BF16."""
    print("case api flux-shaped offload", flush=True)
    import types
    import bench_extra
    a = types.SimpleNamespace(double_blocks=2, single_blocks=3, image_tokens=4096, text_tokens=512)
    report = bench_extra.flux_report(a, torch, torch.device(DEV), passes=4)
    assert report["config"]["parameters"] == 2 * 339_738_624 + 3 * 141_557_760
    assert report["outputs_bit_identical"] == {"resident_vs_bf16": True, "offload_vs_resident": True}
    off, res = report["passes"]["df11_offload"], report["passes"]["df11_resident"]
    assert off["peak_device_memory_mb"] < res["peak_device_memory_mb"]
    M._prefetcher.reset()
    M.TensorManager.clear()
    torch.cuda.empty_cache()


def test_offloaded_model_is_collected_without_reset(tmp_path):
    """An offloaded model that is deleted takes its pinned host streams with it, and the
    prefetcher lets go of the device staging slots it kept for it (no manual reset())."""
    print("case api offload, model deleted", flush=True)
    import gc
    import weakref
    compress_model(make_model(8), PATTERNS, str(tmp_path), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path), device=DEV, bfloat16_model=make_model(9), cpu_offload=True)
    ids = torch.randint(0, 97, (2, 8), device=DEV)
    want = _reference_logits(8, ids)
    with torch.no_grad():
        for _ in range(3):
            assert torch.equal(model(ids), want)
    dev = torch.device(DEV)
    assert M._prefetcher.live.get(dev) == 5 and any(k[0] == dev for k in M._prefetcher.slots)
    layer = weakref.ref(model.layers[1])
    host = weakref.ref(model.layers[1].offloaded_tensors["encoded_exponent"])
    torch.cuda.synchronize()
    del model
    gc.collect()
    assert layer() is None and host() is None
    assert dev not in M._prefetcher.live and not any(k[0] == dev for k in M._prefetcher.slots)
    assert len(M._prefetcher.pending) == 0 and len(M._prefetcher.successor) == 0


def test_streams_rewritten_in_place_are_decoded_anew(tmp_path):
    """load_state_dict copies a second model's streams into the existing buffers: the
    objects stay, their contents change.  The launch arguments and the decode workspace
    derived from the old contents must not be used again."""
    print("case api streams rewritten in place", flush=True)
    from safetensors.torch import load_file
    M._prefetcher.reset()
    a, b = make_model(10), make_model(10)
    with torch.no_grad():
        for p in b.parameters():          # the same values in another order: same code, same stream sizes
            if p.dim() > 1:
                p.copy_(p.flatten().flip(0).view_as(p))
    ref_b = make_model(10)
    ref_b.load_state_dict(b.state_dict())
    compress_model(a, PATTERNS, str(tmp_path / "a"), check_correctness=False)
    compress_model(b, PATTERNS, str(tmp_path / "b"), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path / "a"), device=DEV, bfloat16_model=make_model(9))
    ids = torch.randint(0, 97, (2, 8), device=DEV)
    with torch.no_grad():
        assert torch.equal(model(ids), _reference_logits(10, ids))
        assert torch.equal(model(ids), _reference_logits(10, ids))      # launch arguments bound by now
        state_b = {k: v for k, v in load_file(str(tmp_path / "b" / "model.safetensors")).items()
                   if not k.endswith("split_positions")}
        before = model.layers[0].encoded_exponent
        assert state_b["layers.0.encoded_exponent"].shape == before.shape
        model.load_state_dict(state_b, strict=False)
        assert model.layers[0].encoded_exponent is before               # rewritten in place
        want = ref_b.to(DEV)(ids)
        assert torch.equal(model(ids), want)
        assert torch.equal(model(ids), want)


def test_streams_rebound_to_other_storage_are_decoded_anew(tmp_path):
    """`buffer.data = other` keeps the tensor object and its version counter and points it
    at other memory: the cached launch arguments hold the old addresses and must not be
    used again, nor the workspace derived from the old contents."""
    print("case api streams rebound to other storage", flush=True)
    from safetensors.torch import load_file
    M._prefetcher.reset()
    a, b = make_model(12), make_model(12)
    with torch.no_grad():
        for p in b.parameters():
            if p.dim() > 1:
                p.copy_(p.flatten().flip(0).view_as(p))
    ref_b = make_model(12)
    ref_b.load_state_dict(b.state_dict())
    compress_model(a, PATTERNS, str(tmp_path / "a"), check_correctness=False)
    compress_model(b, PATTERNS, str(tmp_path / "b"), check_correctness=False)
    model = DFloat11Model.from_pretrained(str(tmp_path / "a"), device=DEV, bfloat16_model=make_model(9))
    ids = torch.randint(0, 97, (2, 8), device=DEV)
    with torch.no_grad():
        assert torch.equal(model(ids), _reference_logits(12, ids))
        assert torch.equal(model(ids), _reference_logits(12, ids))      # launch arguments bound by now
        state_b = load_file(str(tmp_path / "b" / "model.safetensors"))
        keep = []                                                       # the old storages stay alive: a stale address would still decode
        for name, module in model.named_modules():
            for key in ("luts", "encoded_exponent", "sign_mantissa", "output_positions", "gaps"):
                full = f"{name}.{key}" if name else key
                if full in state_b and key in module._buffers:
                    buf = module._buffers[key]
                    keep.append(buf.data)
                    version = buf._version
                    buf.data = state_b[full].to(DEV)
                    assert buf._version == version
        want = ref_b.to(DEV)(ids)
        assert torch.equal(model(ids), want)
        assert torch.equal(model(ids), want)


def test_embedding_decodes_only_the_rows_it_looks_up(tmp_path):
    """From its second call on, a compressed nn.Embedding decodes just the rows of its input
    ids: outputs stay bit-identical to the BF16 model's for changing ids (repeated, first and
    last row, non-contiguous views), rows that were not asked for are left as they were in the
    shared buffer, and with the switch off the whole table is decoded as before."""
    print("case api embedding row decode", flush=True)
    import torch.nn as nn
    M._prefetcher.reset()
    M.TensorManager.clear()
    torch.manual_seed(3)
    vocab, dim = 5000, 192

    class Holder(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = nn.Embedding(vocab, dim).to(torch.bfloat16)

        def forward(self, ids):
            return self.embed(ids)

    source = Holder()
    ref_weight = source.embed.weight.detach().clone().to(DEV)
    compress_model(source, {r"embed": []}, str(tmp_path / "e"), check_correctness=False)
    shell = Holder()
    model = DFloat11Model.from_pretrained(str(tmp_path / "e"), device=DEV, bfloat16_model=shell)
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        ids = torch.randint(0, vocab, (4, 16), generator=g).to(DEV)
        assert torch.equal(model(ids), ref_weight[ids])                 # first call: whole table, arguments bound
        buf = M.TensorManager._tensors[torch.device(DEV)]
        for shape in ((1, 1), (3, 7), (4, 16)):
            buf.view(torch.int16).fill_(0x1234)                         # what another module's decode leaves behind
            ids = torch.randint(0, vocab, shape, generator=g).to(DEV)
            ids.view(-1)[0] = 0
            ids.view(-1)[-1] = vocab - 1
            assert torch.equal(model(ids), ref_weight[ids]), shape
            table = model.embed.weight
            untouched = (table.view(torch.int16) == 0x1234).all(dim=1)
            assert int(untouched.sum()) > vocab // 2                    # only the neighbourhood of the rows was decoded
            assert not untouched[ids.view(-1)].any()
        wide = torch.randint(0, vocab, (6, 40), generator=g).to(DEV)
        narrow = wide[:, -1:]                                           # non-contiguous view, as generate() passes
        assert not narrow.is_contiguous()
        assert torch.equal(model(narrow), ref_weight[narrow])
        many = torch.randint(0, vocab, (40, 64), generator=g).to(DEV)   # more than a quarter of the rows: whole table
        buf.view(torch.int16).fill_(0x1234)
        assert torch.equal(model(many), ref_weight[many])
        assert torch.equal(model.embed.weight, ref_weight)
        M.EMBEDDING_ROW_DECODE = False
        try:
            buf.view(torch.int16).fill_(0x1234)
            assert torch.equal(model(ids), ref_weight[ids])
            assert torch.equal(model.embed.weight, ref_weight)
        finally:
            M.EMBEDDING_ROW_DECODE = True
        # a library that has no row decode for the device says so and the hook decodes the whole table
        real = M._decode.launch_rows
        M._decode.launch_rows = lambda *args: False
        try:
            buf.view(torch.int16).fill_(0x1234)
            assert torch.equal(model(ids), ref_weight[ids])
            assert torch.equal(model.embed.weight, ref_weight)
        finally:
            M._decode.launch_rows = real
