"""Compress a local BFloat16 causal language model to DF11.

The command-line counterpart of compress_model for transformers checkpoints,
with the flags of the reference's compression example
(reference: examples/compress_flux1/compress_flux.py:9-41: --model_name_or_path,
--save_path, --save_single_file, --check_correctness, --block_range):

    python -m dfloat11_amd.compress --model_name_or_path /path/to/bf16-model \\
        --save_path /path/to/model-DF11 --check_correctness

The decoder layers are compressed one stream per layer (q, k, v, o, gate, up,
down), the embedding and the output head one stream each.  Other architectures:
call dfloat11_amd.compress_model with a pattern_dict of your own.
"""
import argparse
import sys

from .inference import LLM_PATTERNS


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model_name_or_path", type=str, required=True, help="local directory of the BF16 model")
    ap.add_argument("--save_path", type=str, required=True)
    ap.add_argument("--save_single_file", action="store_true",
                    help="one model.safetensors instead of one file per compressed block")
    ap.add_argument("--check_correctness", action="store_true",
                    help="decode every stream on the GPU and compare it with the original weights")
    ap.add_argument("--block_range", type=int, nargs=2, default=(0, 10000),
                    help="compress only blocks in this range (to split the work over several processes)")
    a = ap.parse_args(argv)

    import torch
    from transformers import AutoModelForCausalLM, AutoTokenizer
    from . import compress_model

    if a.check_correctness and not torch.cuda.is_available():
        sys.exit("--check_correctness decodes on the GPU, and none is available")
    model = AutoModelForCausalLM.from_pretrained(a.model_name_or_path, torch_dtype=torch.bfloat16)
    patterns = {p: list(v) for p, v in LLM_PATTERNS.items()}
    if getattr(model.config, "tie_word_embeddings", False):
        # the head shares the embedding's weight: one stream, decoded by whichever runs
        model.lm_head.weight = torch.nn.Parameter(model.lm_head.weight.detach().clone(), requires_grad=False)
        model.config.tie_word_embeddings = False
    compress_model(model, patterns, a.save_path, block_range=list(a.block_range),
                   save_single_file=a.save_single_file, check_correctness=a.check_correctness)
    try:
        AutoTokenizer.from_pretrained(a.model_name_or_path).save_pretrained(a.save_path)
    except Exception as e:   # a model directory without tokenizer files is still a model
        print(f"tokenizer not copied: {e}", file=sys.stderr)
    print(f"saved DF11 model to {a.save_path}")


if __name__ == "__main__":
    main()
