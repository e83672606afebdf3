"""Training-step time of a randomly initialised Hugging Face GPT-2 on one GPU:
the unfused eager path, torch's SDPA attention, and every swap of
``oslo_amd.transformers`` (``fuse_all``).  The GEMMs are torch's in all three.

    python -m oslo_amd.transformers.example_gpt2_step --layers 4 --hidden 1024 --heads 16 --seq 1024 --batch 8
"""
import argparse
import time

import torch


def build(args, attention):
    from transformers import GPT2Config, GPT2LMHeadModel

    cfg = GPT2Config(n_layer=args.layers, n_head=args.heads, n_embd=args.hidden, vocab_size=args.vocab,
                     n_positions=args.seq, bos_token_id=0, eos_token_id=0)
    torch.manual_seed(0)
    model = GPT2LMHeadModel(cfg)
    model.config._attn_implementation = attention
    return model.to("cuda:0").to(torch.bfloat16).train()


def step_ms(model, ids, steps):
    opt = torch.optim.SGD(model.parameters(), lr=1e-4)

    def step():
        opt.zero_grad(set_to_none=True)
        model(ids, labels=ids).loss.backward()
        opt.step()

    for _ in range(3):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=4)
    ap.add_argument("--hidden", type=int, default=1024)
    ap.add_argument("--heads", type=int, default=16)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--vocab", type=int, default=8192)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--only", choices=["eager", "sdpa", "fused"], help="time one variant only")
    args = ap.parse_args()
    from oslo_amd.transformers import fuse_all

    ids = torch.randint(0, args.vocab, (args.batch, args.seq), device="cuda:0")
    tokens = args.batch * args.seq
    for name in ([args.only] if args.only else ["eager", "sdpa", "fused"]):
        model = build(args, "eager" if name == "fused" else name)
        if name == "fused":
            print("swaps:", fuse_all(model))
        ms = step_ms(model, ids, args.steps)
        print("%-6s %8.2f ms/step %10.0f tokens/s" % (name, ms, tokens / ms * 1e3), flush=True)
        del model
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
