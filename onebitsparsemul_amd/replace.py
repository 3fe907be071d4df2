"""Swap the nn.Linear layers of a model for BinaryLinear_2_4 and account for the memory, as the reference's
model script does for a TinyLlama checkpoint (tests/python/test_model_replace.py:22-56).

    python -m onebitsparsemul_amd.replace [--model-dir DIR] [--device cuda]

With --model-dir the Llama checkpoint in that local directory is loaded (nothing is downloaded); without it a
small randomly initialised Llama of the same architecture is built, which exercises the same code path.
"""
import argparse

import torch
import torch.nn as nn


def set_module(model, name, module):
    """Replace the submodule `name` (dotted path) of `model`. Reference: test_model_replace.py:22-28."""
    parent = model
    parts = name.split(".")
    for part in parts[:-1]:
        parent = getattr(parent, part)
    setattr(parent, parts[-1], module)


def replace_linear_layers(model, skip=()):
    """Every nn.Linear whose shape the packed format admits (in_features % 32 == 0, out_features % 64 == 0) and
    whose name is not in `skip` becomes a BinaryLinear_2_4 holding the 2:4-pruned signs of its weight; a bias is
    carried over. Returns the accounting the reference prints (test_model_replace.py:30-56)."""
    from . import BinaryLinear_2_4
    replaced, kept, weight_params, bias_params = [], [], 0, 0
    for name, module in list(model.named_modules()):
        if not isinstance(module, nn.Linear):
            continue
        out_features, in_features = module.weight.shape
        if name in skip or in_features % 32 != 0 or out_features % 64 != 0:
            kept.append(name)
            continue
        layer = BinaryLinear_2_4(in_features, out_features).to(module.weight.device)
        layer.pack(module.weight.detach())
        weight_params += module.weight.numel()
        if module.bias is not None:
            layer.bias = module.bias
            bias_params += module.bias.numel()
        set_module(model, name, layer)
        replaced.append(name)
    gib = 1024.0 ** 3
    return dict(replaced=replaced, kept=kept, weight_params=weight_params, bias_params=bias_params,
                fp16_weight_gib=weight_params * 16 / 8 / gib, packed_weight_gib=weight_params * 1.5 / 8 / gib)


def _build_model(model_dir, device):
    from transformers import LlamaConfig, LlamaForCausalLM
    if model_dir:
        model = LlamaForCausalLM.from_pretrained(model_dir, local_files_only=True)
    else:
        config = LlamaConfig(vocab_size=4096, hidden_size=512, intermediate_size=1408, num_hidden_layers=2,
                             num_attention_heads=8, num_key_value_heads=4, max_position_embeddings=256)
        model = LlamaForCausalLM(config)
    return model.to(torch.float16).to(device)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model-dir", default=None)
    ap.add_argument("--device", default="cuda")
    args = ap.parse_args(argv)
    model = _build_model(args.model_dir, args.device)
    on_gpu = args.device.startswith("cuda")
    gib = 1024.0 ** 3
    before = torch.cuda.memory_allocated(0) / gib if on_gpu else float("nan")
    stats = replace_linear_layers(model)
    if on_gpu:
        torch.cuda.empty_cache()
    after = torch.cuda.memory_allocated(0) / gib if on_gpu else float("nan")
    print(f"before model:{before} GB")
    print(f"after model:{after} GB")
    print(f"replaced total params {stats['weight_params'] + stats['bias_params']} in {len(stats['replaced'])} layers "
          f"({len(stats['kept'])} nn.Linear kept)")
    print(f"In our theory, before replaced total params cost: {stats['fp16_weight_gib']} GB; "
          f"rest params mem {before - stats['fp16_weight_gib']} GB")
    print(f"In our theory, after replaced total params cost: {stats['packed_weight_gib']} GB; "
          f"rest params mem {after - stats['packed_weight_gib']} GB")
    if on_gpu:
        tokens = torch.randint(0, model.config.vocab_size, (1, 16), device=args.device)
        with torch.no_grad():
            logits = model(tokens).logits
        print(f"forward through the replaced model: logits {tuple(logits.shape)}, finite={bool(torch.isfinite(logits).all())}")
    return stats


if __name__ == "__main__":
    main()
