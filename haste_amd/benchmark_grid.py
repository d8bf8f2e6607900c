"""The reference's benchmark grid (benchmarks/benchmark_lstm.cc:530-555, benchmark_gru.cc)
on this library: batch sizes {1,16,32,64,128} x hidden sizes {128..4096} x input sizes
{64..512}, T = 50 time steps, 10 samples, and the same CSV lines
(`batch_size,hidden_size,input_size,time_ms`), so that the reference's benchmarks/report.py
reads the output unchanged.

  python -m haste_amd.benchmark_grid --cell lstm --mode training --impl haste_amd > a.csv
  python -m haste_amd.benchmark_grid --cell lstm --mode training --impl torch_nn  > b.csv
  python -m haste_amd.benchmark_grid --compare a.csv b.csv

What one sample times follows the reference: inference = ForwardPass::Run (construction
included, benchmark_lstm.cc:307-327); training = forward + the transposes of x, W, R +
BackwardPass::Run (benchmark_lstm.cc:399-465).  `--impl torch_nn` runs torch.nn.LSTM /
torch.nn.GRU on the GPU (the vendor RNN library behind PyTorch-ROCm), where the reference
runs cuDNN: forward, or forward + backward with the same upstream gradients.
"""
import argparse
import sys

import numpy as np

BATCH_SIZES = (1, 16, 32, 64, 128)
HIDDEN_SIZES = (128, 256, 512, 768, 1024, 1536, 2048, 3072, 4096)
INPUT_SIZES = (64, 128, 256, 512)


def time_ms(torch, fn, samples):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(samples):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / samples


def haste_sample(torch, ops, cell, training, T, N, C, H):
    dev = torch.device("cuda")
    G = 4 if cell == "lstm" else 3
    x = torch.rand(T, N, C, device=dev)
    W, R = torch.rand(C, G * H, device=dev) - 0.5, (torch.rand(H, G * H, device=dev) - 0.5) * H ** -0.5
    b, b2 = torch.rand(G * H, device=dev), torch.rand(G * H, device=dev)
    z = torch.zeros(N, H, device=dev)
    dh, dc = torch.rand(T + 1, N, H, device=dev), torch.rand(T + 1, N, H, device=dev)
    no_mask = torch.empty(0, 0, 0, device=dev)
    if cell == "lstm":
        def fwd():
            return ops.lstm_forward(training, 0.0, x, z, z, W, R, b, no_mask)

        def train():
            h, c, cache = fwd()
            ops.lstm_backward(ops.transpose(x), ops.transpose(W), ops.transpose(R), b, no_mask, h, c,
                              cache, dh, dc)
    else:
        def fwd():
            return ops.gru_forward(training, 0.0, x, z, W, R, b, b2, no_mask)

        def train():
            h, cache = fwd()
            ops.gru_backward(ops.transpose(x), ops.transpose(W), ops.transpose(R), b, b2, no_mask, h,
                             cache, dh)
    return train if training else fwd


def torch_nn_sample(torch, cell, training, T, N, C, H):
    dev = torch.device("cuda")
    layer = (torch.nn.LSTM if cell == "lstm" else torch.nn.GRU)(C, H).to(dev)
    x = torch.rand(T, N, C, device=dev, requires_grad=training)
    dy = torch.rand(T, N, H, device=dev)
    if not training:
        layer.eval()

        def fwd():
            with torch.no_grad():
                return layer(x)
        return fwd

    def train():
        layer.zero_grad(set_to_none=True)
        x.grad = None
        y, _ = layer(x)
        y.backward(dy)
    return train


def compare(path_a, path_b):
    A, B = np.loadtxt(path_a, delimiter=",", ndmin=2), np.loadtxt(path_b, delimiter=",", ndmin=2)
    # Keep the grid points both files hold (a run cut short still compares).
    in_b = {tuple(r[:3]): r for r in B}
    A = np.array([r for r in A if tuple(r[:3]) in in_b])
    if len(A) == 0:
        sys.exit("the two files share no grid point")
    B = np.array([in_b[tuple(r[:3])] for r in A])
    faster = 1.0 - A[:, -1] / B[:, -1]
    print("A is faster than B by:  mean %.1f%%  median %.1f%%  min %.1f%%  max %.1f%%  "
          "(A faster on %d of %d points)" % (100 * faster.mean(), 100 * np.median(faster),
                                             100 * faster.min(), 100 * faster.max(),
                                             int((faster > 0).sum()), len(faster)))
    print("time A / time B, geometric mean over the input sizes:")
    hs = sorted(set(A[:, 1]))
    print("batch \\ hidden " + " ".join("%7d" % h for h in hs))
    for n in sorted(set(A[:, 0])):
        cells = []
        for h in hs:
            sel = (A[:, 0] == n) & (A[:, 1] == h)
            cells.append("%7.2f" % np.exp(np.mean(np.log(A[sel, -1] / B[sel, -1]))))
        print("%14d " % n + " ".join(cells))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--cell", choices=["lstm", "gru"], default="lstm")
    ap.add_argument("--mode", choices=["inference", "training"], default="training")
    ap.add_argument("--impl", choices=["haste_amd", "torch_nn"], default="haste_amd")
    ap.add_argument("--sample_size", type=int, default=10)
    ap.add_argument("--time_steps", type=int, default=50)
    ap.add_argument("--batch_sizes", type=int, nargs="+", default=list(BATCH_SIZES))
    ap.add_argument("--hidden_sizes", type=int, nargs="+", default=list(HIDDEN_SIZES))
    ap.add_argument("--input_sizes", type=int, nargs="+", default=list(INPUT_SIZES))
    ap.add_argument("--compare", nargs=2, metavar=("A.csv", "B.csv"))
    args = ap.parse_args()
    if args.compare:
        compare(*args.compare)
        return
    import torch
    from haste_amd import ops
    training = args.mode == "training"
    print("# Benchmark configuration:")
    print("#   Mode: %s" % args.mode)
    print("#   Implementation: %s (%s)" % (args.impl, args.cell))
    print("#   Sample size: %d" % args.sample_size)
    print("#   Time steps: %d" % args.time_steps)
    print("#")
    print("# batch_size,hidden_size,input_size,time_ms")
    for N in args.batch_sizes:
        for H in args.hidden_sizes:
            for C in args.input_sizes:
                if args.impl == "haste_amd":
                    fn = haste_sample(torch, ops, args.cell, training, args.time_steps, N, C, H)
                else:
                    fn = torch_nn_sample(torch, args.cell, training, args.time_steps, N, C, H)
                print("%d,%d,%d,%f" % (N, H, C, time_ms(torch, fn, args.sample_size)), flush=True)


if __name__ == "__main__":
    main()
