"""Model shapes of the decode workloads (the five benchmark configurations)."""
from collections import namedtuple

Shape = namedtuple("Shape", "name nLayers dim nHeads nKVHeads headDim ffnDim vocab eps theta bias tied fmt")


def _s(name, L, dim, H, KV, hd, ffn, vocab, eps, theta, bias, tied, fmt):
    return Shape(name, L, dim, H, KV, hd, ffn, vocab, eps, theta, bias, tied, fmt)


TOY = _s("toy", 4, 512, 8, 8, 64, 1376, 256, 1e-5, 1e4, False, True, "q8")
QWEN = _s("qwen2.5-0.5b", 24, 896, 14, 2, 64, 4864, 151936, 1e-6, 1e6, True, True, "q8")
TINYLLAMA = _s("tinyllama-1.1b", 22, 2048, 32, 4, 64, 5632, 32000, 1e-5, 1e4, False, False, "q8")
QWEN_Q4 = _s("qwen2.5-0.5b-q4_0", 24, 896, 14, 2, 64, 4864, 151936, 1e-6, 1e6, True, False, "q4_0")
LLAMA3_8B = _s("llama-3-8b", 32, 4096, 32, 8, 128, 14336, 128256, 1e-5, 5e5, False, False, "q8")

BY_NAME = {s.name: s for s in (TOY, QWEN, TINYLLAMA, QWEN_Q4, LLAMA3_8B)}


def kv_dim(s):
    return s.nKVHeads * s.headDim


def weight_bytes_per_token(s):
    """Weights + per-row scales + norm gains read once per token (biases and
    activations excluded), the figure the bandwidth roofline uses."""
    kv = kv_dim(s)

    def mat(n, k):
        return n * k + 4 * n if s.fmt == "q8" else n * (k // 32) * 18

    per_layer = 2 * mat(s.dim, s.dim) + 2 * mat(kv, s.dim) + 2 * mat(s.ffnDim, s.dim) + mat(s.dim, s.ffnDim) + 8 * s.dim
    return s.nLayers * per_layer + mat(s.vocab, s.dim) + 4 * s.dim


def kv_bytes_at(s, pos):
    return 2 * s.nLayers * (pos + 1) * kv_dim(s) * 4
