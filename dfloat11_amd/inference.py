"""Generation benchmark: tokens per second and GPU memory of a DF11 model,
optionally against the same model in BF16.

Flags follow the reference's benchmark script (reference: inference.py:10-17:
--model_name_or_path, --bf16, --prompt, --num_tokens, --batch_size, --seed) and
the report has the same fields (latency, tokens per second, allocated and peak
GPU memory: inference.py:75-97).  Without network access there are no
checkpoints to download, so `--synthetic SHAPE` builds the named architecture
locally with random-init N(0, 0.02) BF16 weights and compresses it in memory
(same encoder, same buffers and hooks as a model loaded from DF11 safetensors).

    python -m dfloat11_amd.inference --synthetic qwen3-8b --num_tokens 256 \
        --batch_size 1 --prompt_len 64 --compare_bf16
    python -m dfloat11_amd.inference --model_name_or_path /path/to/df11-model
"""
import argparse
import json
import re
import sys
import time

LLM_PATTERNS = {
    r"model\.embed_tokens": [],
    r"lm_head": [],
    r"model\.layers\.\d+": [
        "self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
        "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj",
    ],
}

SHAPES = {
    # hidden, intermediate, layers, heads, kv heads, head_dim, vocab, tied embeddings
    "qwen3-8b": dict(arch="qwen3", hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
                     num_attention_heads=32, num_key_value_heads=8, head_dim=128, vocab_size=151936,
                     tie_word_embeddings=True),
    "llama-3-8b": dict(arch="llama", hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                       num_attention_heads=32, num_key_value_heads=8, head_dim=128, vocab_size=128256,
                       tie_word_embeddings=False),
    "tiny": dict(arch="qwen3", hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                 num_attention_heads=4, num_key_value_heads=2, head_dim=64, vocab_size=1024,
                 tie_word_embeddings=True),
}


def build_synthetic(shape, device, seed, layers=None):
    """Random-init model of a named shape, BF16, on `device`."""
    import torch
    from transformers import AutoModelForCausalLM, LlamaConfig, Qwen3Config
    spec = dict(SHAPES[shape])
    arch = spec.pop("arch")
    if layers:
        spec["num_hidden_layers"] = layers
    cfg_cls = Qwen3Config if arch == "qwen3" else LlamaConfig
    cfg = cfg_cls(max_position_embeddings=4096, initializer_range=0.02, **spec)
    torch.manual_seed(seed)
    with torch.device(device):
        model = AutoModelForCausalLM.from_config(cfg, torch_dtype=torch.bfloat16)
    return model.eval()


def convert_in_memory(model, pattern_dict, device, cpu_offload=False, pin_memory=True):
    """Replaces the weights selected by `pattern_dict` with DF11 streams on
    `device`, without going through files: what compress_model followed by
    DFloat11Model.from_pretrained leaves behind (reference: dfloat11.py:496-598
    and 179-308).  With cpu_offload the two large streams of every module stay in
    (pinned) host memory, as load_and_replace_tensors arranges them.  Weights
    shared between modules (tied embeddings) are compressed once per module that
    uses them.  Returns (compressed bytes, BF16 bytes)."""
    import torch
    import torch.nn as nn
    from . import dfloat11 as D
    from .dfloat11_utils import encode_weights, get_32bit_codec, get_codec, get_luts

    hook = D.get_hook(D.threads_per_block, D.bytes_per_thread)
    compressed = original = 0
    for pattern, attr_names in pattern_dict.items():
        for full_name, sub_module in list(model.named_modules()):
            if not re.fullmatch(pattern, full_name):
                continue
            if isinstance(sub_module, (nn.Embedding, nn.Linear)):
                targets = [sub_module]
            else:
                targets = [sub_module.get_submodule(a) for a in attr_names]
            weights = [t.weight.data.detach().to("cpu").flatten() for t in targets]
            _, counter = get_codec(torch.cat(weights))
            codec, _, table = get_32bit_codec(counter)
            encoded, other_8bits, output_positions, gaps, split_positions = encode_weights(
                weights, codec, D.bytes_per_thread, D.threads_per_block[0])
            for t in targets:
                D._drop_weight(t)
            del weights
            tensors = {"luts": get_luts(table), "encoded_exponent": encoded, "sign_mantissa": other_8bits,
                       "output_positions": output_positions.view(torch.uint8), "gaps": gaps}
            for key, value in tensors.items():
                compressed += value.numel() * value.element_size()
                if cpu_offload and key in D.offloaded_tensor_names:
                    if not hasattr(sub_module, "offloaded_tensors"):
                        sub_module.offloaded_tensors = {}
                    sub_module.offloaded_tensors[key] = value.pin_memory() if pin_memory else value
                else:
                    sub_module.register_buffer(key, value.to(device))
            original += other_8bits.numel() * 2
            sub_module.split_positions = split_positions.tolist()
            if not isinstance(sub_module, (nn.Embedding, nn.Linear)):
                sub_module.weight_injection_modules = targets
            sub_module.register_forward_pre_hook(hook)
    if hasattr(model, "config"):
        model.config.dfloat11_config = {"version": D.version, "threads_per_block": D.threads_per_block,
                                        "bytes_per_thread": D.bytes_per_thread, "pattern_dict": pattern_dict}
    return compressed, original


def timed_generate(model, inputs, num_tokens, do_sample):
    """Reference: inference.py:62-74."""
    import torch
    torch.cuda.reset_peak_memory_stats()
    torch.cuda.synchronize()
    with torch.no_grad():
        start = time.time()
        output = model.generate(**inputs, max_new_tokens=num_tokens, min_new_tokens=num_tokens,
                                do_sample=do_sample)
        torch.cuda.synchronize()
        latency = time.time() - start
    n_new = output.shape[1] - inputs["input_ids"].shape[1]
    return output, {
        "latency_s": latency,
        "new_tokens_per_sequence": n_new,
        "tokens_per_second": n_new * output.shape[0] / latency,
        "gpu_memory_allocated_mb": torch.cuda.memory_allocated() / 1e6,
        "gpu_peak_memory_mb": torch.cuda.max_memory_allocated() / 1e6,
    }


def _random_prompts(model, batch_size, prompt_len, seed, device):
    import torch
    gen = torch.Generator(device="cpu").manual_seed(seed)
    ids = torch.randint(0, model.config.vocab_size, (batch_size, prompt_len), generator=gen).to(device)
    return {"input_ids": ids, "attention_mask": torch.ones_like(ids)}


def compare_synthetic(shape, batch_sizes, num_tokens, prompt_len=64, seed=42, device="cuda:0", layers=None,
                      repeats=1):
    """Builds the named architecture once with random-init BF16 weights, compresses a copy
    of it in memory, and generates greedily from the same prompts with both at every batch
    size.  Returns one report per batch size with the fields of the reference's benchmark
    for both models (reference: inference.py:62-97), their ratio, and whether logits and
    tokens are identical.  The timed runs of the two models alternate (BF16, DF11, BF16, ...,
    `repeats` of each) and each model reports its run of median latency: generation speed of
    the eager model drifts by several per cent over a minute on the same box, and runs taken
    one model after the other would put that drift into the ratio.  Both models are resident
    throughout, so each model's memory figures are what the device holds minus the other
    model's share."""
    import copy
    import torch
    device = torch.device(device)
    model = build_synthetic(shape, device, seed, layers)
    name = f"{shape} (random-init N(0, 0.02), {sum(p.numel() for p in model.parameters())/1e9:.2f} B parameters)"
    bf16_bytes = torch.cuda.memory_allocated(device)
    df11_model = copy.deepcopy(model)
    t0 = time.time()
    compressed, original = convert_in_memory(df11_model, LLM_PATTERNS, device)
    compress_seconds = time.time() - t0
    torch.cuda.empty_cache()
    reports = []
    for b in batch_sizes:
        inputs = _random_prompts(model, b, prompt_len, seed, device)
        with torch.no_grad():
            ref_logits = model(**inputs, use_cache=False).logits
            # also the DF11 model's warm-up pass: first-use work (decode workspaces, library
            # handles) stays out of the timing
            logits = df11_model(**inputs, use_cache=False).logits
        logits_identical = bool(torch.equal(logits, ref_logits))
        del logits, ref_logits
        timed_generate(model, inputs, min(8, num_tokens), False)
        timed_generate(df11_model, inputs, min(8, num_tokens), False)
        df11_bytes = torch.cuda.memory_allocated(device) - bf16_bytes      # streams, shared buffer, workspaces
        runs = {"bf16": [], "df11": []}
        for _ in range(max(1, repeats)):
            runs["bf16"].append(timed_generate(model, inputs, num_tokens, False))
            runs["df11"].append(timed_generate(df11_model, inputs, num_tokens, False))
        report = {"batch_size": b, "num_tokens": num_tokens, "model": name, "prompt_len": prompt_len,
                  "compress_seconds": compress_seconds, "compressed_over_bf16": compressed / original,
                  "logits_bit_identical": logits_identical}
        outs = {}
        for which, other_bytes in (("bf16", df11_bytes), ("df11", bf16_bytes)):
            ordered = sorted(runs[which], key=lambda r: r[1]["latency_s"])
            outs[which], stats = ordered[len(ordered) // 2]
            stats = dict(stats, timed_runs=len(ordered))
            for key in ("gpu_memory_allocated_mb", "gpu_peak_memory_mb"):
                stats[key] -= other_bytes / 1e6
            report[which] = stats
        report["tokens_identical"] = bool(torch.equal(outs["df11"], outs["bf16"]))
        report["df11_over_bf16_tokens_per_second"] = (report["df11"]["tokens_per_second"]
                                                      / report["bf16"]["tokens_per_second"])
        reports.append(report)
    del model, df11_model
    from . import dfloat11 as D
    D.TensorManager.clear()
    torch.cuda.empty_cache()
    return reports


def _print_report(report, as_json):
    if as_json:
        print(json.dumps(report))
        return
    for key, value in report.items():
        if isinstance(value, dict):
            print(f"[{key}]")
            print(f"  Decoding Latency for {value['new_tokens_per_sequence']} tokens: {value['latency_s']:.4f} seconds")
            print(f"  Tokens per second: {value['tokens_per_second']:.2f}")
            print(f"  GPU Memory Allocated: {value['gpu_memory_allocated_mb']:.2f} MB")
            print(f"  GPU Peak Memory Usage: {value['gpu_peak_memory_mb']:.2f} MB")
        else:
            print(f"{key}: {value}")


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model_name_or_path", type=str, default=None)
    ap.add_argument("--bf16", action="store_true", help="the model at --model_name_or_path is plain BFloat16")
    ap.add_argument("--prompt", type=str, default="Question: What is a binary tree and its applications? Answer:")
    ap.add_argument("--num_tokens", type=int, default=1024)
    ap.add_argument("--batch_size", type=int, default=1)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--synthetic", choices=sorted(SHAPES), default=None,
                    help="build this architecture with random weights instead of loading a checkpoint")
    ap.add_argument("--layers", type=int, default=None, help="override the number of layers of --synthetic")
    ap.add_argument("--prompt_len", type=int, default=64, help="random prompt token ids per sequence (--synthetic)")
    ap.add_argument("--greedy", action="store_true", help="greedy decoding (default for --synthetic)")
    ap.add_argument("--compare_bf16", action="store_true",
                    help="--synthetic only: run the BF16 model first, then its DF11 form, and compare")
    ap.add_argument("--repeats", type=int, default=1,
                    help="--compare_bf16 only: timed generations per model, alternating; the median run is reported")
    ap.add_argument("--device", type=str, default="cuda:0")
    ap.add_argument("--json", action="store_true", help="print one JSON line instead of the text report")
    a = ap.parse_args(argv)

    import torch
    from transformers import set_seed
    if not torch.cuda.is_available():
        sys.exit("a GPU is required: DF11 weights are decoded on the GPU only")
    device = torch.device(a.device)
    torch.cuda.set_device(device)
    report = {"batch_size": a.batch_size, "num_tokens": a.num_tokens}

    if a.synthetic and a.compare_bf16:
        report = compare_synthetic(a.synthetic, [a.batch_size], a.num_tokens, a.prompt_len, a.seed, device,
                                   a.layers, a.repeats)[0]
        _print_report(report, a.json)
        return report
    if a.synthetic:
        model = build_synthetic(a.synthetic, device, a.seed, a.layers)
        inputs = _random_prompts(model, a.batch_size, a.prompt_len, a.seed, device)
        do_sample = False
        report["model"] = f"{a.synthetic} (random-init N(0, 0.02), {sum(p.numel() for p in model.parameters())/1e9:.2f} B parameters)"
        report["prompt_len"] = a.prompt_len
        t0 = time.time()
        compressed, original = convert_in_memory(model, LLM_PATTERNS, device)
        report["compress_seconds"] = time.time() - t0
        report["compressed_over_bf16"] = compressed / original
        torch.cuda.empty_cache()
    else:
        if not a.model_name_or_path:
            sys.exit("give --model_name_or_path (a local directory) or --synthetic")
        from transformers import AutoModelForCausalLM, AutoTokenizer
        if a.bf16:
            model = AutoModelForCausalLM.from_pretrained(a.model_name_or_path, torch_dtype=torch.bfloat16).to(device)
        else:
            from . import DFloat11Model
            model = DFloat11Model.from_pretrained(a.model_name_or_path, device=str(device))
        tokenizer = AutoTokenizer.from_pretrained(a.model_name_or_path)
        tokenizer.pad_token = tokenizer.eos_token
        tokenizer.padding_side = "left"
        inputs = dict(tokenizer([a.prompt] * a.batch_size, return_tensors="pt", padding=True).to(device))
        do_sample = not a.greedy
        report["model"] = a.model_name_or_path

    # warm-up pass: first-use work (decode workspaces, library handles) stays out of the timing
    with torch.no_grad():
        logits = model(**inputs, use_cache=False).logits
    set_seed(a.seed)
    timed_generate(model, inputs, min(8, a.num_tokens), do_sample)
    set_seed(a.seed)
    out, stats = timed_generate(model, inputs, a.num_tokens, do_sample)
    report["bf16_model" if (a.bf16 and not a.synthetic) else "df11"] = stats

    _print_report(report, a.json)
    return report


if __name__ == "__main__":
    main()
