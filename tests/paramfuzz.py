"""Mutated .param texts for the parser: characters deleted, replaced and doubled, tokens that parsers trip over spliced in,
the text cut short; and the same nets in the binary .param form with words replaced by awkward values, dropped, doubled,
bytes flipped, the file cut short.  load_param / load_param_bin have to answer every one of them with a return code (and
load_model, where the net still loads, with an error at the latest when it finds no GPU) -- never with a crash.  Run in a
child process by the test."""
import sys

import numpy as np


def bases():
    from ncnn_amd import modelwriter as mw, zoo
    g, tiny_param, blob, info = zoo.build("tiny")
    gemm = mw.assemble_param(["Input in0 0 1 a 0=96 1=24", "Input in1 0 1 b 0=96 1=40", "Input in2 0 1 c 0=40",
                              mw.gemm_param("g", ["a", "b", "c"], "out", constantB=0, alpha=0.5),
                              mw.gemm_param("g2", ["out"], "out2", N=16, K=40, constantB=1, quantize_term=801),
                              mw.innerproduct_param("fc", "out2", "out3", 8, 128, 1, 2, 1), "Pooling pool 1 1 out3 out4 0=1 1=3 11=2 2=2 12=1 3=1 5=2 6=0"])
    mha = mw.assemble_param(["Input in_q 0 1 q 0=64 1=4", "Input in_m 0 1 m", "Input in_ck 0 1 ck", "Input in_cv 0 1 cv",
                             mw.mha_param("mha", ["q", "m", "ck", "cv"], ["out", "ko", "vo"], 64, 4, 64, attn_mask=1, kv_cache=1, quantize_term=801)])
    return [tiny_param, gemm, mha], blob


TOKENS = ["0=", "1=", "-23310=", "=", " ", "\n", "7767517", "-1", "99999999999", "1e40", "nan", "0=1,2,3", "-23300=5,1,2", "-23310=-5,1", "Convolution", "Split",
          "x" * 300, "\0", "-", "2147483648", "-2147483649", "0x10", "1 1", "0 0", "\t", "-23301=99999999"]


def mutate(rng, text):
    s = list(text)
    for _ in range(int(rng.integers(1, 6))):
        kind = rng.integers(5)
        pos = int(rng.integers(0, len(s) + 1))
        if kind == 0 and s:
            del s[pos % len(s)]
        elif kind == 1:
            s[pos:pos] = list(TOKENS[int(rng.integers(len(TOKENS)))])
        elif kind == 2 and s:
            s[pos % len(s)] = chr(int(rng.integers(32, 127)))
        elif kind == 3:
            s = s[:pos]
        elif kind == 4 and s:
            a = pos % len(s)
            b = min(len(s), a + int(rng.integers(1, 40)))
            s[a:b] = s[a:b] * 2
    return "".join(s)


def main(seed, count):
    from ncnn_amd import host
    texts, blob = bases()
    rng = np.random.default_rng(seed)
    loaded = 0
    for it in range(count):
        text = mutate(rng, texts[it % len(texts)])
        net = host.Net()
        net.register_int8_layers()
        net.register_attention_layer()
        if net.load_param_mem(text) == 0:
            loaded += 1
            net.load_model_mem(blob)
    print("survived %d mutated texts, %d of them still loaded" % (count, loaded))


WORDS = [0, -1, 1, 2, 255, 256, 257, 1 << 24, (1 << 24) + 1, 2 ** 31 - 1, -2 ** 31, -233, -23300, -23301, -23310, -23330, -23400, -23401, -23431, 32, 31,
         6, 15, 16, 42, 74, 79, 7767517]


def mutate_bin(rng, data):
    w = list(np.frombuffer(data[: len(data) // 4 * 4], "<i4"))
    for _ in range(int(rng.integers(1, 5))):
        kind, pos = int(rng.integers(5)), int(rng.integers(0, len(w) + 1))
        if kind == 0 and w:
            w[pos % len(w)] = WORDS[int(rng.integers(len(WORDS)))]
        elif kind == 1 and w:
            del w[pos % len(w)]
        elif kind == 2:
            w = w[:pos]
        elif kind == 3 and w:
            a = pos % len(w)
            b = min(len(w), a + int(rng.integers(1, 12)))
            w[a:b] = w[a:b] * 2
        elif kind == 4 and w:
            w[pos % len(w)] = int(np.int32(np.uint32(int(w[pos % len(w)]) & 0xFFFFFFFF) ^ np.uint32(1 << int(rng.integers(32)))))
    out = np.array(w, "<i4").tobytes()
    return out[: len(out) - int(rng.integers(4))] if rng.random() < 0.2 else out


def main_bin(seed, count):
    import os
    import tempfile
    from ncnn_amd import host, modelwriter as mw
    texts, blob = bases()
    bins = [mw.assemble_param_bin(t.splitlines()[2:])[0] for t in texts]
    rng = np.random.default_rng(seed)
    loaded = 0
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "net.param.bin")  # through a file: the memory form of the call has no length to stop at
        for it in range(count):
            with open(path, "wb") as f:
                f.write(mutate_bin(rng, bins[it % len(bins)]))
            net = host.Net()
            net.register_int8_layers()
            net.register_attention_layer()
            if net.load_param_bin(path) == 0:
                loaded += 1
                net.load_model_mem(blob)
    print("survived %d mutated binary params, %d of them still loaded" % (count, loaded))


if __name__ == "__main__":
    (main_bin if len(sys.argv) > 3 and sys.argv[3] == "bin" else main)(int(sys.argv[1]), int(sys.argv[2]))
