"""Text generation through the "moba" attention plugin on an MI355X.

Counterpart of the reference's example (examples/llama.py:6-36) with the same switches
(--model, --moba-chunk-size, --moba-topk, --attn).  A model directory on disk is loaded with
transformers; with --random-weights a small Llama (head_dim 128, grouped-query heads) is built
from a local config instead, so the whole path -- registration, HIP prefill, HIP decode --
runs without any download.

    python examples/generate.py --random-weights --prompt-tokens 6000 --moba-chunk-size 512 --moba-topk 4
    python examples/generate.py --model /path/to/Llama-3.1-8B --attn moba
"""

import argparse
import os
import sys
import time

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from moba_amd import MoBAConfig, register_moba  # noqa: E402


def build_model(args, dtype):
    from transformers import AutoModelForCausalLM, LlamaConfig, LlamaForCausalLM
    if args.random_weights:
        cfg = LlamaConfig(vocab_size=32000, hidden_size=1024, intermediate_size=2816, num_hidden_layers=4,
                          num_attention_heads=8, num_key_value_heads=2, head_dim=128,
                          max_position_embeddings=max(8192, args.prompt_tokens + args.new_tokens + 8))
        torch.manual_seed(0)
        model = LlamaForCausalLM(cfg).to(dtype)
    else:
        model = AutoModelForCausalLM.from_pretrained(args.model, torch_dtype=dtype)
    model.config._attn_implementation = args.attn
    return model.to("cuda").eval()


def prompt_ids(args, model):
    if args.random_weights or args.prompt is None:
        g = torch.Generator().manual_seed(1)
        return torch.randint(0, model.config.vocab_size, (1, args.prompt_tokens), generator=g).to("cuda"), None
    from transformers import AutoTokenizer
    tok = AutoTokenizer.from_pretrained(args.model)
    return torch.tensor([tok.encode(args.prompt)], device="cuda"), tok


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", default=None, help="directory of a transformers causal LM (no downloads are attempted)")
    ap.add_argument("--random-weights", action="store_true", help="small random-weight Llama built locally")
    ap.add_argument("--moba-chunk-size", type=int, default=4096)
    ap.add_argument("--moba-topk", type=int, default=12)
    ap.add_argument("--attn", default="moba", choices=["moba", "moba_naive", "sdpa", "eager"])
    ap.add_argument("--full-attention-layers", type=int, nargs="*", default=None,
                    help="decoder layers that use full attention (negative = from the end)")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    ap.add_argument("--prompt", default=None)
    ap.add_argument("--prompt-tokens", type=int, default=4096, help="length of the random prompt")
    ap.add_argument("--new-tokens", type=int, default=16)
    args = ap.parse_args()
    if not args.random_weights and args.model is None:
        ap.error("give --model DIR or --random-weights")

    register_moba(MoBAConfig(args.moba_chunk_size, args.moba_topk, full_attention_layers=args.full_attention_layers))
    model = build_model(args, getattr(torch, args.dtype))
    ids, tok = prompt_ids(args, model)
    with torch.no_grad():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = model.generate(ids, max_new_tokens=args.new_tokens, do_sample=False)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    new = out[0, ids.shape[1]:].tolist()
    print(f"attn={args.attn} prompt={ids.shape[1]} tokens, {len(new)} new tokens in {dt * 1e3:.1f} ms")
    print(tok.decode(new) if tok is not None else new)


if __name__ == "__main__":
    main()
