"""Writes tests/golden/cfg1_seed0.json: the small MoE layer of BASELINE configs[0] at seed 0, computed by the CPU
oracle (oracle/zbal_oracle.cpp). The reference holds no vectors for this path, so this is a regression fixture of
this repository's own definition: routing indices and layout in full, SHA-256 digests of the bulk tensors plus
their leading values. Run from the repository root:  python tests/golden/make_cfg1_fixture.py"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as zo  # noqa: E402


def cfg1_inputs():
    T, H, E, K, N = 256, 1024, 8, 2, 2048
    g = np.random.default_rng(0)
    x = zo.f32_to_bf16(g.standard_normal((T, H)).astype(np.float32))
    logits = g.standard_normal((T, E)).astype(np.float32)
    wf = (g.standard_normal((E, H, N)) * 0.02).astype(np.float32)
    wscale = (np.abs(wf).max(axis=1) / 127.0).astype(np.float32)
    w = np.clip(np.rint(wf / wscale[:, None, :]), -127, 127).astype(np.int8)
    return dict(T=T, H=H, E=E, K=K, N=N, x=x, logits=logits, w=w, wscale=wscale)


def cfg1_oracle(c):
    idx, tw = zo.topk_route(c["logits"], c["K"])
    _, per_expert, send = zo.dispatch_layout(idx, c["E"], 1)
    put = np.concatenate([[0], np.cumsum(per_expert)[:-1]]).astype(np.int32)
    q, s = zo.dispatch_normal(c["x"], zo.DT_BF16, idx.astype(np.int32), send, put, c["E"], 1, c["T"] * c["K"])
    y = zo.grouped_gemm_w8a8_dequant(q, s, c["w"], c["wscale"], per_expert.astype(np.int64))
    out = zo.combine(y, zo.DT_BF16, put, tw, idx.astype(np.int32), send, c["E"])
    return dict(topk_idx=idx, topk_w=tw, tokens_per_expert=per_expert, put_offset=put, send_token_idx=send, q=q,
                scale=s, y=y, out=out)


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    c = cfg1_inputs()
    r = cfg1_oracle(c)
    fx = {
        "config": {k: c[k] for k in ("T", "H", "E", "K", "N")},
        "inputs_sha256": {k: digest(c[k]) for k in ("x", "logits", "w", "wscale")},
        "topk_idx": r["topk_idx"].tolist(),
        "tokens_per_expert": r["tokens_per_expert"].tolist(),
        "put_offset": r["put_offset"].tolist(),
        "sha256": {k: digest(r[k]) for k in ("topk_w", "send_token_idx", "q", "scale", "y", "out")},
        "head": {"topk_w": r["topk_w"][:4].tolist(), "q_row0": r["q"][0, :16].tolist(),
                 "scale": r["scale"][:4].astype(np.float64).tolist(), "y_row0_bits": r["y"][0, :8].tolist(),
                 "out_row0_bits": r["out"][0, :8].tolist()},
    }
    path = os.path.join(ROOT, "tests", "golden", "cfg1_seed0.json")
    with open(path, "w") as f:
        json.dump(fx, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
