"""Swap the nn.Linear layers of a model for BinaryLinear_2_4 and account for the memory, as the reference's
model script does for a TinyLlama checkpoint (tests/python/test_model_replace.py:22-56).

    python -m onebitsparsemul_amd.replace [--model-dir DIR] [--device cuda] [--time]
    python -m onebitsparsemul_amd.replace --hidden 4096 --intermediate 11008 --layers 2 --time

With --model-dir the Llama checkpoint in that local directory is loaded (nothing is downloaded); without it a
small randomly initialised Llama of the same architecture is built (its sizes can be set), which exercises the same
code path. --time also measures the forward pass over 16 and 512 tokens before and after the replacement.
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


def _build_model(model_dir, device, hidden=512, intermediate=1408, layers=2):
    from transformers import LlamaConfig, LlamaForCausalLM
    if model_dir:
        model = LlamaForCausalLM.from_pretrained(model_dir, local_files_only=True)
    else:
        heads = max(1, hidden // 64)
        config = LlamaConfig(vocab_size=4096, hidden_size=hidden, intermediate_size=intermediate,
                             num_hidden_layers=layers, num_attention_heads=heads,
                             num_key_value_heads=max(1, heads // 2), max_position_embeddings=1024)
        model = LlamaForCausalLM(config)
    return model.to(torch.float16).to(device)


def _forward_ms(model, tokens, repeats=20):
    """Average time of one forward pass over `tokens` (1 x T token ids), in milliseconds."""
    with torch.no_grad():
        for _ in range(3):
            model(tokens)
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(repeats):
            model(tokens)
        stop.record()
        torch.cuda.synchronize()
    return start.elapsed_time(stop) / repeats


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model-dir", default=None)
    ap.add_argument("--device", default="cuda")
    ap.add_argument("--hidden", type=int, default=512, help="hidden size of the randomly initialised model")
    ap.add_argument("--intermediate", type=int, default=1408)
    ap.add_argument("--layers", type=int, default=2)
    ap.add_argument("--time", action="store_true", help="time the forward pass before and after (GPU only)")
    args = ap.parse_args(argv)
    model = _build_model(args.model_dir, args.device, args.hidden, args.intermediate, args.layers)
    on_gpu = args.device.startswith("cuda")
    gib = 1024.0 ** 3
    timed = {}
    if on_gpu and args.time:
        for count in (16, 512):
            ids = torch.randint(0, model.config.vocab_size, (1, count), device=args.device)
            timed[count] = [ids, _forward_ms(model, ids)]
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
        for count, (ids, before_ms) in timed.items():
            print(f"forward over {count} tokens: {before_ms:.3f} ms with nn.Linear (fp16), "
                  f"{_forward_ms(model, ids):.3f} ms with BinaryLinear_2_4")
    return stats


if __name__ == "__main__":
    main()
