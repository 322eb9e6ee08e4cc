"""Autotunes ten everyday operators written as Tensor Comprehensions, each from the naive
mapping options, and times the winner next to PyTorch's own routine on the same GPU.

    python examples/tune_common_operators.py [name,name,...] [generations x population, default 5x40]

Prints one line per operator: kernel time of the tuned TC (and the HBM rate where the operator is
memory-bound), the library's time, the largest relative difference between the two results, the
tuning wall time, the launch shapes and the options found."""
import os
import sys
import time

import torch
import torch.nn.functional as F

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import tensorcomprehensions_amd as tc  # noqa: E402


def microseconds(fn, launches=30):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(5):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(launches):
            fn()
        stop.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(stop) * 1e3 / launches)
    return best


def rand(*shape):
    return torch.randn(*shape, device="cuda")


# name -> (TC text, inputs, library routine, bytes moved when memory-bound else 0)
OPERATORS = {
    "layernorm": ("""def layernorm(float(M, N) X, float(N) g, float(N) b) -> (mean, var, Y) {
        mean(m) +=! X(m, n) / N
        var(m) +=! (X(m, n) - mean(m)) * (X(m, n) - mean(m)) / N
        Y(m, n) = (X(m, n) - mean(m)) * rsqrt(var(m) + 0.00001) * g(n) + b(n) }""",
                  lambda: [rand(8192, 4096), rand(4096), rand(4096)],
                  lambda x, g, b: F.layer_norm(x, (4096,), g, b), 2 * 8192 * 4096 * 4),
    "bmm": ("def bmm(float(B, M, K) X, float(B, K, N) Y) -> (Z) { Z(b, m, n) +=! X(b, m, k) * Y(b, k, n) }",
            lambda: [rand(64, 512, 64), rand(64, 64, 512)], torch.bmm, 0),
    "conv3x3": ("""def conv(float(N, C, H, W) I, float(M, C, KH, KW) W1) -> (O) {
        O(n, m, h, w) +=! I(n, c, h + kh, w + kw) * W1(m, c, kh, kw) }""",
                lambda: [rand(32, 64, 58, 58), rand(64, 64, 3, 3)], F.conv2d, 0),
    "transpose": ("def to_channels_last(float(N, C, H, W) I) -> (O) { O(n, h, w, c) = I(n, c, h, w) }",
                  lambda: [rand(32, 256, 56, 56)], lambda i: i.permute(0, 2, 3, 1).contiguous(), 2 * 32 * 256 * 56 * 56 * 4),
    "gemv": ("def gemv(float(M, K) A, float(K) x) -> (y) { y(m) +=! A(m, k) * x(k) }",
             lambda: [rand(16384, 8192), rand(8192)], lambda a, x: a @ x, 16384 * 8192 * 4),
    "softmax": ("""def softmax(float(M, N) X) -> (mx, s, Y) {
        mx(m) max=! X(m, n)
        s(m) +=! exp(X(m, n) - mx(m))
        Y(m, n) = exp(X(m, n) - mx(m)) / s(m) }""",
                lambda: [rand(8192, 4096)], lambda x: torch.softmax(x, 1), 2 * 8192 * 4096 * 4),
    "maxpool2x2": ("""def maxpool(float(N, C, H, W) I) -> (O) {
        O(n, c, h, w) max=! I(n, c, 2 * h + kh, 2 * w + kw) where kh in 0:2, kw in 0:2 }""",
                   lambda: [rand(32, 64, 112, 112)], lambda i: F.max_pool2d(i, 2), 5 * 32 * 64 * 56 * 56 * 4),
    "depthwise3x3": ("""def depthwise(float(N, C, H, W) I, float(C, KH, KW) W1) -> (O) {
        O(n, c, h, w) +=! I(n, c, h + kh, w + kw) * W1(c, kh, kw) }""",
                     lambda: [rand(32, 128, 58, 58), rand(128, 3, 3)],
                     lambda i, w: F.conv2d(i, w.unsqueeze(1), groups=128), 32 * 128 * (58 * 58 + 56 * 56) * 4),
    "embedding": ("def embedding(float(V, E) T, int32(B) idx) -> (O) { O(b, e) = T(idx(b), e) }",
                  lambda: [rand(50000, 1024), torch.randint(0, 50000, (16384,), device="cuda", dtype=torch.int32)],
                  lambda t, i: F.embedding(i, t), 2 * 16384 * 1024 * 4),
    "bias_gradient": ("def bias_gradient(float(N, M, H, W) d_O) -> (d_B) { d_B(m) +=! d_O(n, m, h, w) }",
                      lambda: [rand(32, 64, 56, 56)], lambda d: d.sum((0, 2, 3)), 32 * 64 * 56 * 56 * 4),
}


def main():
    names = sys.argv[1].split(",") if len(sys.argv) > 1 and sys.argv[1] != "all" else list(OPERATORS)
    generations, population = (int(v) for v in (sys.argv[2] if len(sys.argv) > 2 else "5x40").split("x"))
    for name in names:
        text, make_inputs, library, nbytes = OPERATORS[name]
        entry = text.split("(")[0].split()[1]
        inputs = make_inputs()
        outputs = tc.prepare_outputs(text, entry, inputs)
        outputs = list(outputs) if isinstance(outputs, (list, tuple)) else [outputs]
        t0 = time.time()
        best = tc.autotune(text, entry, inputs, "naive", outputs=outputs, generations=generations, pop_size=population,
                           threads=16, seed=1, top_k=1)
        tuning = time.time() - t0
        executor = tc.compile(text, entry, inputs, best[0])
        t_tc = microseconds(lambda: tc.unchecked_run(executor, inputs, outputs))
        t_lib = microseconds(lambda: library(*inputs))
        reference = library(*inputs)
        torch.cuda.synchronize()
        error = (outputs[-1] - reference).abs().max().item() / max(1.0, reference.abs().max().item())
        rate = f" ({nbytes / t_tc / 1e6:.2f} TB/s)" if nbytes else ""
        launches = [executor.launch_bounds(k) for k in range(executor.num_kernels)]
        options = best[0].to_text()
        print(f"{name}: TC {t_tc:.1f} us{rate} | library {t_lib:.1f} us | relative difference {error:.1e} | "
              f"tuned in {tuning:.0f} s | {launches}\n    {options[options.find('tile='):]}", flush=True)


if __name__ == "__main__":
    main()
