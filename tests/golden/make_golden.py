#!/usr/bin/env python3
"""Writes the committed fixtures under tests/golden/.  Run in the authoring container only (it reads the
reference's published result logs under /root/reference and uses CPU torch as an independent implementation):

    python tests/golden/make_golden.py

Fixtures (data only):
    reference_logs.json    per-request CPU_Time / CUDA_Time columns and the printed totals of the reference's two
                           published runs (Baseline_Result.txt, Liger_Result.txt) -- the known-answer test of the
                           report arithmetic (src/schedule.h:325-348)
    fill_normal_words.json first outputs of the counter-based generator from an independent numpy restatement
    cfg1_layer_torch.npz   output of one BASELINE-config-1 layer (hidden 256, 4 x 64 heads, FFN 1024, batch 2, seq 32,
                           fp32, seed 0) in both norm modes, computed with torch ops (matmul, softmax, layer_norm,
                           gelu(tanh)) from inputs drawn with the numpy restatement of the generator
"""
import json
import os
import re
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference"


def splitmix(z):
    with np.errstate(over="ignore"):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def fill_normal(n, seed, tid, mean=0.0, std=1.0):
    """numpy restatement of the generator (integer Irwin-Hall(8), two rounded fp32 operations)."""
    with np.errstate(over="ignore"):
        key = splitmix(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(tid))
        i = np.arange(n, dtype=np.uint64)
        a = splitmix(key + np.uint64(2) * i)
        b = splitmix(key + np.uint64(2) * i + np.uint64(1))

    def s4(r):
        return ((r & np.uint64(0xFFFF)) + ((r >> np.uint64(16)) & np.uint64(0xFFFF)) + ((r >> np.uint64(32)) & np.uint64(0xFFFF))
                + (r >> np.uint64(48))).astype(np.int64)

    s = (s4(a) + s4(b) - 262140).astype(np.float32)
    z = s * np.float32(float.fromhex("0x1.3988e2p-16"))
    return (np.float32(std) * z + np.float32(mean)).astype(np.float32)


def parse_log(path):
    cpu, gpu, totals = [], [], {}
    for line in open(path):
        m = re.match(r"request: (\d+), CPU_Time: ([\d.eE+-]+) ms, CUDA_Time: ([\d.eE+-]+) ms", line)
        if m:
            cpu.append(float(m.group(2)))
            gpu.append(float(m.group(3)))
        for key in ("Total_Duration", "Throughput", "Average Latency"):
            m = re.match(key + r": ([\d.eE+-]+)", line)
            if m:
                totals[key] = float(m.group(1))
        m = re.match(r"Total (\d+) records", line)
        if m:
            totals["records"] = int(m.group(1))
    return {"cpu_ms": cpu, "gpu_ms": gpu, "printed": totals}


def cfg1_weights():
    H, h, d, F = 256, 4, 64, 1024
    spec = [("wq", (H, H), 0.02, 0), ("wk", (H, H), 0.02, 0), ("wv", (H, H), 0.02, 0), ("bq", (H,), 0.02, 0), ("bk", (H,), 0.02, 0),
            ("bv", (H,), 0.02, 0), ("wo", (H, H), 0.02, 0), ("bo", (H,), 0.02, 0), ("ln1_g", (H,), 0.1, 1), ("ln1_b", (H,), 0.1, 0),
            ("w1", (H, F), 0.02, 0), ("b1", (F,), 0.02, 0), ("w2", (F, H), 0.02, 0), ("b2", (H,), 0.02, 0), ("ln2_g", (H,), 0.1, 1),
            ("ln2_b", (H,), 0.1, 0)]
    w = {}
    for tid, (name, shape, std, mean) in enumerate(spec, start=1):
        w[name] = fill_normal(int(np.prod(shape)), 0, tid, mean, std).reshape(shape)
    x = fill_normal(2 * 32 * H, 0, 99).reshape(64, H)
    return w, x


def torch_layer(w, x, norm_mode, B=2, S=32, h=4, d=64):
    import torch
    import torch.nn.functional as Fn
    t = {k: torch.from_numpy(v).double() for k, v in w.items()}
    x = torch.from_numpy(x).double()
    H = h * d

    def ln(v, g, b):
        return Fn.layer_norm(v, (H,), g, b, eps=1e-6)

    def mha(v):
        q = (v @ t["wq"] + t["bq"]).view(B, S, h, d).transpose(1, 2)
        k = (v @ t["wk"] + t["bk"]).view(B, S, h, d).transpose(1, 2)
        vv = (v @ t["wv"] + t["bv"]).view(B, S, h, d).transpose(1, 2)
        sc = (q @ k.transpose(-1, -2)) / (d ** 0.5)
        e = torch.exp(sc - sc.max(-1, keepdim=True).values)
        p = e / (e.sum(-1, keepdim=True) + 1e-6)  # the reference's +1e-6 denominator
        o = (p @ vv).transpose(1, 2).reshape(B * S, H)
        return o @ t["wo"]

    def mlp(v):
        return Fn.gelu(v @ t["w1"] + t["b1"], approximate="tanh") @ t["w2"]

    if norm_mode == 0:  # MHA -> LN -> MLP -> LN, no residuals, no out/FFN-2 bias  (src/layer/bert.h:59-79)
        a = mha(x)
        l = ln(a, t["ln1_g"], t["ln1_b"])
        return ln(mlp(l), t["ln2_g"], t["ln2_b"]).float().numpy()
    n1 = ln(x, t["ln1_g"], t["ln1_b"])
    a = mha(n1) + x + t["bo"]
    n2 = ln(a, t["ln2_g"], t["ln2_b"])
    return (mlp(n2) + a + t["b2"]).float().numpy()


def main():
    logs = {"baseline": parse_log(os.path.join(REF, "Baseline_Result.txt")), "liger": parse_log(os.path.join(REF, "Liger_Result.txt"))}
    json.dump(logs, open(os.path.join(HERE, "reference_logs.json"), "w"))
    words = {"seed0_tid1_n8": [float(v) for v in fill_normal(8, 0, 1)],
             "seed7_tid42_mean0.25_std0.02_n8": [float(v) for v in fill_normal(8, 7, 42, 0.25, 0.02)],
             "seed0_tid1_at_1000000": float(fill_normal(1000001, 0, 1)[-1])}
    json.dump(words, open(os.path.join(HERE, "fill_normal_words.json"), "w"), indent=1)
    w, x = cfg1_weights()
    np.savez_compressed(os.path.join(HERE, "cfg1_layer_torch.npz"), post_noresid=torch_layer(w, x, 0), pre_ln_resid=torch_layer(w, x, 1))
    print("fixtures written to", HERE)


if __name__ == "__main__":
    sys.exit(main())
