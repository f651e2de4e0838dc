"""Command-line driver of the end-to-end sparse attention model, with the options of the reference's script
(end2end/sspmm_e2e/end_to_end.py:20-35) and its measurement (10 forward passes to warm up, 32 timed, :194-203),
here with a device synchronisation either side of the timed loop.

    python -m sspmm_amd.end_to_end --seq_len 4096 --embed_dim 256 --num_heads 4 --sparsity 0.9 --bs 8 --model both

`--model dense` runs the same architecture with torch's dense attention (the reference's comparison model,
end_to_end.py:79-121 and 151-175); `--mem` reports the peak device memory of one forward pass instead of a time;
`--graph` also replays the forward pass from a HIP graph.
"""
import argparse
import time

import torch

from .attention import SparseAttentionEncoder


def _parser():
    p = argparse.ArgumentParser(description="Sparse multi-head attention encoder, forward pass")
    p.add_argument("--vocab_size", type=int, default=257)
    p.add_argument("--num_class", type=int, default=2, help="accepted for compatibility; the head is mlp_dim wide as in the reference's driver")
    p.add_argument("--mlp_dim", type=int, default=1024)
    p.add_argument("--embed_dim", type=int, default=256, help="head_dim * num_heads")
    p.add_argument("--num_heads", type=int, default=4)
    p.add_argument("--bs", type=int, default=2, help="batch size")
    p.add_argument("--seq_len", type=int, default=4096)
    p.add_argument("--sparsity", type=float, default=0.9, help="share of the mask's vectors that are left out")
    p.add_argument("--vec_length", type=int, default=8, choices=(8, 16))
    p.add_argument("--model", choices=("sparse", "dense", "both"), default="sparse")
    p.add_argument("--mem", action="store_true", help="report the peak device memory of a forward pass")
    p.add_argument("--graph", action="store_true", help="also time the forward pass replayed from a HIP graph")
    p.add_argument("--seed", type=int, default=0)
    return p


class _DenseAttention(torch.nn.Module):
    """The model's blocks with torch's dense attention on the same weights."""

    def __init__(self, model):
        super().__init__()
        self.model = model

    def forward(self, tokens):
        m = self.model
        seq, bsz = tokens.size(1), tokens.size(0)
        out = m.encoder(tokens) * (m.embed_dim ** 0.5)
        out = out.transpose(0, 1) + m.pe[:seq].to(out.dtype)
        for blk in m.blocks:
            h, d = blk.num_heads, m.embed_dim // blk.num_heads
            q, k, v = blk.in_proj(blk.layer_norm1(out)).chunk(3, dim=-1)
            q, k, v = (t.contiguous().view(seq, bsz * h, d).transpose(0, 1) for t in (q, k, v))
            a = torch.nn.functional.scaled_dot_product_attention(q, k, v).transpose(0, 1).contiguous().view(seq, bsz, m.embed_dim)
            h1 = blk.out_proj(a) + out
            out = blk.linear2(blk.linear1(blk.layer_norm2(h1))) + out
        return m.linear(m.layer_norm(out))


def _time(fn, warm=10, timed=32):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(timed):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / timed * 1e3


def _graphed(fn):
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        fn()
    return g.replay


def main(argv=None):
    args = _parser().parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("sspmm_amd.end_to_end needs a GPU")
    if args.embed_dim % args.num_heads or args.seq_len % args.vec_length:
        raise SystemExit("embed_dim must be a multiple of num_heads and seq_len of vec_length")
    torch.manual_seed(args.seed)
    model = SparseAttentionEncoder(args.vocab_size, args.embed_dim, args.num_heads, args.sparsity, args.seq_len, args.mlp_dim,
                                   args.mlp_dim, vec_length=args.vec_length, layers=4, seed=args.seed).cuda().half().eval()
    tokens = torch.randint(0, args.vocab_size, (args.bs, args.seq_len), device="cuda")
    runs = []
    if args.model in ("sparse", "both"):
        runs.append(("vectorSparse", lambda: model(tokens)))
    if args.model in ("dense", "both"):
        dense = _DenseAttention(model)
        runs.append(("dense", lambda: dense(tokens)))
    with torch.no_grad():
        for name, fn in runs:
            if args.mem:
                torch.cuda.reset_peak_memory_stats()
                fn()
                torch.cuda.synchronize()
                print("%s peak memory %.1f MB, batchsize [%d]" % (name, torch.cuda.max_memory_allocated() / 2 ** 20, args.bs))
                continue
            print("%s average runtime %.4f milliseconds, batchsize [%d]" % (name, _time(fn), args.bs))
            if args.graph:
                print("%s average runtime %.4f milliseconds from a graph, batchsize [%d]" % (name, _time(_graphed(fn)), args.bs))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
