"""Write the golden vectors under tests/golden/ by running the reference once.

Run from the repository root, in the build container only (the reference does
not exist anywhere else):

    python tests/golden/make_fixtures.py [/root/reference [step ...]]

The script imports the reference package from the given checkout, feeds it
seeded synthetic inputs and stores inputs + outputs as .npz / .json data.  The
rotation matrix Pi always travels as data: torch.linalg.qr is not bitwise
reproducible across BLAS thread counts, so no test regenerates it on one side
of a comparison only.

bf16 / fp16 tensors are stored as their raw 16-bit patterns (suffix `_bits`)
together with a dtype tag, because numpy has no bfloat16.
"""

from __future__ import annotations

import hashlib
import json
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.dont_write_bytecode = True      # leave no __pycache__ behind in the read-only reference tree
sys.path.insert(0, REF)

import turboquant.codebook as ref_codebook          # noqa: E402
from turboquant.quantizer import (                  # noqa: E402
    TurboQuantProd, TurboQuantMSE, MSEQuantized, _pack_indices, _unpack_indices,
)
from turboquant.rotation import rotate_forward      # noqa: E402
from turboquant.kv_cache import quantize_values, dequantize_values, TurboQuantKVCache  # noqa: E402
from turboquant.store import CompressedKVStore      # noqa: E402
from turboquant.capture import KVCaptureEngine      # noqa: E402
from turboquant.score import compute_hybrid_attention  # noqa: E402

CPU = torch.device("cpu")


def bits16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().copy()


def store_float(out: dict, name: str, t: torch.Tensor):
    if t.dtype in (torch.bfloat16, torch.float16):
        out[name + "_bits"] = bits16(t)
        out[name + "_dtype"] = np.array("bf16" if t.dtype == torch.bfloat16 else "fp16")
    else:
        out[name] = t.contiguous().numpy().copy()


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(t.contiguous().numpy().tobytes()).hexdigest()


def seed_codebook_cache(d: int, bits: int):
    """Keep get_codebook from writing a JSON into the reference tree for a
    (d, bits) pair it does not ship."""
    key = (d, bits)
    path = os.path.join(REF, "turboquant", "codebooks", f"codebook_d{d}_b{bits}.json")
    if key not in ref_codebook._CODEBOOK_CACHE and not os.path.exists(path):
        ref_codebook._CODEBOOK_CACHE[key] = ref_codebook.compute_lloyd_max_codebook(d, bits)
    return ref_codebook.get_codebook(d, bits)


def key_trace(tq: TurboQuantProd, x: torch.Tensor):
    """Quantise through the reference and also expose the two intermediate
    tensors the packing consumes (rotated unit vectors y, projected residual p),
    recomputed with the reference's own calls in the reference's own order."""
    code = tq.quantize(x)
    mq = tq.mse_quantizer
    norms = x.norm(dim=-1, keepdim=False)
    unit = x / (norms.unsqueeze(-1) + 1e-10)
    y = rotate_forward(unit.float(), mq.Pi)
    x_hat = mq.dequantize(MSEQuantized(indices=code.mse_indices, norms=code.norms, bits=code.mse_bits))
    p = torch.matmul((x - x_hat).float(), tq.S.T)
    return code, y, p


# ---------------------------------------------------------------- config 1
def config1():
    g = torch.Generator(device="cpu").manual_seed(0)
    K = torch.randn(4096, 128, generator=g, dtype=torch.float32)
    K = K / K.norm(dim=-1, keepdim=True)
    K = K * (0.5 + 1.5 * torch.rand(4096, generator=g)).unsqueeze(-1)
    Q = torch.randn(32, 128, generator=g, dtype=torch.float32)
    Q = Q / Q.norm(dim=-1, keepdim=True)
    Q = Q * (0.5 + 1.5 * torch.rand(32, generator=g)).unsqueeze(-1)

    tq = TurboQuantProd(128, bits=3, device=CPU)
    t0 = time.perf_counter()
    code, y, p = key_trace(tq, K)
    scores = tq.attention_score(Q, code)
    wall = time.perf_counter() - t0
    deq = tq.dequantize(code)

    out = {
        "Pi": tq.mse_quantizer.Pi.numpy(), "S": tq.S.numpy(),
        "centroids": tq.mse_quantizer.centroids.numpy(),
        "thresholds": tq.mse_quantizer.decision_boundaries.numpy(),
        "mse_indices": code.mse_indices.numpy(), "qjl_signs": code.qjl_signs.numpy(),
        "norms": code.norms.numpy(), "residual_norms": code.residual_norms.numpy(),
        "scores": scores.numpy(),
        # a slice of the intermediates, enough for the bit-exact packing check
        "y_head": y[:256].numpy(), "p_head": p[:256].numpy(), "deq_head": deq[:64].numpy(),
        "K_head": K[:256].numpy(), "Q": Q.numpy(),
    }
    np.savez_compressed(os.path.join(HERE, "config1_full.npz"), **out)
    digest = {
        "K_sha256": sha(K), "Q_sha256": sha(Q),
        "mse_indices_sha256": sha(code.mse_indices), "qjl_signs_sha256": sha(code.qjl_signs),
        "scores_rms": float(scores.pow(2).mean().sqrt()),
        "torch": torch.__version__, "threads": torch.get_num_threads(),
        "reference_wall_s": wall,
    }
    with open(os.path.join(HERE, "config1_digest.json"), "w") as f:
        json.dump(digest, f, indent=1)
    print("config1:", digest)


# ---------------------------------------------------------------- keys, 16-bit inputs and other widths
def key_cases():
    out = {}
    cases = [
        ("bf16_d128_b3", 128, 3, torch.bfloat16, 11),
        ("fp16_d128_b3", 128, 3, torch.float16, 12),
        ("fp32_d128_b4", 128, 4, torch.float32, 13),
        ("bf16_d64_b2", 64, 2, torch.bfloat16, 14),
        ("bf16_d256_b3", 256, 3, torch.bfloat16, 15),
        ("fp32_d64_b5", 64, 5, torch.float32, 16),
    ]
    for name, d, bits, dt, seed in cases:
        seed_codebook_cache(d, bits - 1)
        g = torch.Generator(device="cpu").manual_seed(seed)
        x = torch.randn(2, 48, d, generator=g, dtype=torch.float32)
        ch = torch.randperm(d, generator=g)[:4]
        x[..., ch] *= 20.0
        x[0, 0] = 0.0                      # an all-zero vector exercises the +1e-10 guard
        x = x.to(dt)
        q = torch.randn(2, 5, d, generator=g, dtype=torch.float32).to(dt)
        tq = TurboQuantProd(d, bits=bits, device=CPU, seed=42 + 7 * (seed % 3))
        code, y, p = key_trace(tq, x)
        store_float(out, f"{name}.x", x)
        store_float(out, f"{name}.q", q)
        out[f"{name}.Pi"] = tq.mse_quantizer.Pi.numpy()
        out[f"{name}.S"] = tq.S.numpy()
        out[f"{name}.centroids"] = tq.mse_quantizer.centroids.numpy()
        out[f"{name}.thresholds"] = tq.mse_quantizer.decision_boundaries.numpy()
        out[f"{name}.y"] = y.numpy()
        out[f"{name}.p"] = p.numpy()
        out[f"{name}.mse_indices"] = code.mse_indices.numpy()
        out[f"{name}.qjl_signs"] = code.qjl_signs.numpy()
        store_float(out, f"{name}.norms", code.norms)
        out[f"{name}.residual_norms"] = code.residual_norms.numpy()
        out[f"{name}.dequant"] = tq.dequantize(code).numpy()
        out[f"{name}.scores"] = tq.attention_score(q, code).numpy()
        out[f"{name}.meta"] = np.array([d, bits, 42 + 7 * (seed % 3)])
    np.savez_compressed(os.path.join(HERE, "key_cases.npz"), **out)
    print("key_cases:", len(out), "arrays")


# ---------------------------------------------------------------- keys, wide heads and the zero-coordinate bucket
def key_cases_wide():
    """head_dim 576 with 4-bit keys (the only d = 576 table the reference ships is the 3-bit one) and
    head_dim 128 with 5-bit keys: the two shipped tables whose middle threshold is a tiny negative number
    instead of 0, so that the all-zero vector in each case lands in the upper middle bucket.  The sketch
    matrix S is not stored for d = 576 (1.3 MB): it is torch.randn of seed + 1000, which is bit-stable."""
    out = {}
    for name, d, bits, dt, seed, n_tok in (("bf16_d576_b4", 576, 4, torch.bfloat16, 17, 24),
                                           ("bf16_d128_b5", 128, 5, torch.bfloat16, 18, 48)):
        seed_codebook_cache(d, bits - 1)
        g = torch.Generator(device="cpu").manual_seed(seed)
        x = torch.randn(2, n_tok, d, generator=g, dtype=torch.float32)
        ch = torch.randperm(d, generator=g)[:4]
        x[..., ch] *= 20.0
        x[0, 0] = 0.0
        x[1, 3] = 0.0
        x = x.to(dt)
        q = torch.randn(2, 5, d, generator=g, dtype=torch.float32).to(dt)
        tq = TurboQuantProd(d, bits=bits, device=CPU, seed=42 + 7 * (seed % 3))
        code, y, p = key_trace(tq, x)
        store_float(out, f"{name}.x", x)
        store_float(out, f"{name}.q", q)
        out[f"{name}.Pi"] = tq.mse_quantizer.Pi.numpy()
        if d <= 256:
            out[f"{name}.S"] = tq.S.numpy()
        out[f"{name}.centroids"] = tq.mse_quantizer.centroids.numpy()
        out[f"{name}.thresholds"] = tq.mse_quantizer.decision_boundaries.numpy()
        out[f"{name}.y"] = y.numpy()
        out[f"{name}.p"] = p.numpy()
        out[f"{name}.mse_indices"] = code.mse_indices.numpy()
        out[f"{name}.qjl_signs"] = code.qjl_signs.numpy()
        store_float(out, f"{name}.norms", code.norms)
        out[f"{name}.residual_norms"] = code.residual_norms.numpy()
        out[f"{name}.dequant"] = tq.dequantize(code).numpy()
        out[f"{name}.scores"] = tq.attention_score(q, code).numpy()
        out[f"{name}.meta"] = np.array([d, bits, 42 + 7 * (seed % 3)])
    np.savez_compressed(os.path.join(HERE, "key_cases_wide.npz"), **out)
    print("key_cases_wide:", len(out), "arrays")


# ---------------------------------------------------------------- packing
def packing():
    out = {}
    g = torch.Generator(device="cpu").manual_seed(21)
    for bits in (1, 2, 3, 4, 5):
        for d in (128, 13):
            idx = torch.randint(0, 2 ** bits, (7, d), generator=g)
            pk = _pack_indices(idx, bits)
            out[f"idx_b{bits}_d{d}"] = idx.numpy()
            out[f"packed_b{bits}_d{d}"] = pk.numpy()
            out[f"unpacked_b{bits}_d{d}"] = _unpack_indices(pk, bits, d).numpy()
    tq = TurboQuantProd(64, bits=2, device=CPU)
    for d in (64, 13):
        proj = torch.randn(5, d, generator=g)
        proj[0, :3] = 0.0
        out[f"proj_d{d}"] = proj.numpy()
        out[f"signs_d{d}"] = tq._pack_qjl_signs(proj).numpy()
    out["signs_unpacked_d64"] = tq._unpack_qjl_signs(torch.from_numpy(out["signs_d64"])).numpy()
    np.savez_compressed(os.path.join(HERE, "packing.npz"), **out)
    print("packing:", len(out), "arrays")


# ---------------------------------------------------------------- values
def values():
    out = {}
    for dt, tag in ((torch.bfloat16, "bf16"), (torch.float16, "fp16"), (torch.float32, "fp32")):
        for bits in (2, 4, 8):
            for gs in (32, 64):
                g = torch.Generator(device="cpu").manual_seed(31 + bits + gs)
                v = torch.randn(3, 32, 128, generator=g, dtype=torch.float32)
                v[0, 0, :32] = 1.25          # a constant group exercises the 1e-10 scale clamp
                v[1, :, 5] *= 20.0
                v = v.to(dt)
                vq = quantize_values(v, bits=bits, group_size=gs)
                name = f"{tag}_b{bits}_g{gs}"
                store_float(out, f"{name}.v", v)
                out[f"{name}.data"] = vq.data.numpy()
                store_float(out, f"{name}.scales", vq.scales)
                store_float(out, f"{name}.zeros", vq.zeros)
                out[f"{name}.dequant"] = dequantize_values(vq, gs).numpy()
    np.savez_compressed(os.path.join(HERE, "values.npz"), **out)
    print("values:", len(out), "arrays")


# ---------------------------------------------------------------- codebooks: shipped data files + d=256
def codebooks_d256():
    src = os.path.join(REF, "turboquant", "codebooks")
    for fn in sorted(os.listdir(src)):
        if fn.endswith(".json"):            # data files the reference ships: known answers for the solver
            with open(os.path.join(src, fn)) as f:
                cb = json.load(f)
            with open(os.path.join(HERE, "ref_" + fn), "w") as f:
                json.dump(cb, f, indent=2)
    for bits in (1, 2, 3):
        cb = ref_codebook.compute_lloyd_max_codebook(256, bits)
        with open(os.path.join(HERE, f"ref_codebook_d256_b{bits}.json"), "w") as f:
            json.dump(cb, f, indent=2)
        print("codebook d256 b", bits, cb["mse_total"])


# ---------------------------------------------------------------- hybrid attention through store + capture engine
def hybrid():
    out = {}
    H, G, d = 2, 2, 128
    for name, n_hist, n_recent, vb in (("hist72_ring128", 72, 128, 2), ("hist200_only", 200, 0, 4),
                                       ("ring40_only", 0, 40, 2), ("hist8_ring5", 8, 5, 2), ("hist48_ring3_b4", 48, 3, 4)):
        g = torch.Generator(device="cpu").manual_seed(41 + n_hist)
        store = CompressedKVStore(d, H, key_bits=3, value_bits=vb, value_group_size=32, device=CPU, layer_idx=3)
        q = torch.randn(1, H * G, d, generator=g).to(torch.bfloat16)
        if n_hist:
            k = torch.randn(n_hist, H, d, generator=g).to(torch.bfloat16)
            v = torch.randn(n_hist, H, d, generator=g).to(torch.bfloat16)
            store.append_chunk(k[: n_hist // 2], v[: n_hist // 2])
            store.append_chunk(k[n_hist // 2:], v[n_hist // 2:])
            store_float(out, f"{name}.k", k)
            store_float(out, f"{name}.v", v)
            flat = store.get_flat_cache()
            out[f"{name}.mse_indices"] = flat.prod_q.mse_indices.numpy()
            out[f"{name}.qjl_signs"] = flat.prod_q.qjl_signs.numpy()
            store_float(out, f"{name}.norms", flat.prod_q.norms)
            out[f"{name}.residual_norms"] = flat.prod_q.residual_norms.numpy()
            out[f"{name}.v_data"] = flat.value_q.data.numpy()
            store_float(out, f"{name}.v_scales", flat.value_q.scales)
            store_float(out, f"{name}.v_zeros", flat.value_q.zeros)
            out[f"{name}.memory_bytes"] = np.array(store.memory_bytes())
        rk = rv = None
        if n_recent:
            rk = torch.randn(n_recent, H, d, generator=g).to(torch.bfloat16)
            rv = torch.randn(n_recent, H, d, generator=g).to(torch.bfloat16)
            store_float(out, f"{name}.recent_k", rk)
            store_float(out, f"{name}.recent_v", rv)
        res = compute_hybrid_attention(q, store, rk, rv, num_query_heads=H * G)
        store_float(out, f"{name}.q", q)
        store_float(out, f"{name}.out", res)
        out[f"{name}.Pi"] = store.quantizer.mse_quantizer.Pi.numpy()
        out[f"{name}.S"] = store.quantizer.S.numpy()
        out[f"{name}.meta"] = np.array([H, G, d, n_hist, n_recent, vb])
    np.savez_compressed(os.path.join(HERE, "hybrid.npz"), **out)
    print("hybrid:", len(out), "arrays")


# ---------------------------------------------------------------- capture policy trace
class _TagStore:
    """Duck-typed stand-in for the store: records which token tags arrive."""

    def __init__(self, heads, dim):
        self.num_kv_heads, self.head_dim, self.device = heads, dim, CPU
        self.chunks = []

    @property
    def num_tokens(self):
        return sum(len(c) for c in self.chunks)

    def append_chunk(self, key, value):
        self.chunks.append([int(t) for t in key[:, 0, 0].float().tolist()])

    def reset(self):
        self.chunks = []


def capture_trace():
    traces = []
    for cap, prefill, decodes, flush in ((8, 5, 30, True), (8, 8, 9, False), (8, 21, 17, True), (128, 300, 260, False),
                                         (4, 0, 13, True)):
        st = _TagStore(2, 8)
        eng = KVCaptureEngine(st, ring_capacity=cap, device=CPU, dtype=torch.float32)   # fp32 keeps the token tags exact
        tok = 0
        if prefill:
            k = torch.arange(prefill, dtype=torch.float32).view(-1, 1, 1).expand(prefill, 2, 8)
            eng.ingest_prefill(k, k, prefill)
            tok = prefill
        for _ in range(decodes):
            k = torch.full((1, 2, 8), float(tok))
            eng.ingest_decode(k, k, 1)
            tok += 1
        if flush:
            eng.flush()
        peek = eng.ring.peek()
        ring = [] if peek is None else [int(t) for t in peek[0][:, 0, 0].float().tolist()]
        traces.append({"capacity": cap, "prefill": prefill, "decodes": decodes, "flush": flush,
                       "chunks": st.chunks, "ring": ring,
                       "total_compressed": eng.total_compressed_tokens, "total_buffered": eng.total_buffered_tokens,
                       "ring_total_written": eng.ring.total_written})
    # a second prefill into a non-empty ring: the overflow is dropped (capture.py:176-180)
    st = _TagStore(1, 4)
    eng = KVCaptureEngine(st, ring_capacity=4, device=CPU)
    a = torch.arange(3, dtype=torch.float32).view(-1, 1, 1).expand(3, 1, 4).to(torch.bfloat16)
    b = (10 + torch.arange(3, dtype=torch.float32)).view(-1, 1, 1).expand(3, 1, 4).to(torch.bfloat16)
    eng.ingest_prefill(a, a, 3)
    eng.ingest_prefill(b, b, 3)
    peek = eng.ring.peek()
    traces.append({"capacity": 4, "double_prefill": True, "chunks": st.chunks,
                   "ring": [int(t) for t in peek[0][:, 0, 0].float().tolist()]})
    with open(os.path.join(HERE, "capture_trace.json"), "w") as f:
        json.dump(traces, f)
    print("capture_trace:", len(traces), "cases")


# ---------------------------------------------------------------- stand-alone cache object
def kv_cache_object():
    out = {}
    g = torch.Generator(device="cpu").manual_seed(51)
    cache = TurboQuantKVCache(128, key_bits=3, value_bits=2, buffer_size=16, device=CPU, dtype=torch.float32, layer_idx=1)
    k = torch.randn(1, 2, 40, 128, generator=g)
    v = torch.randn(1, 2, 40, 128, generator=g)
    cache.prefill(k, v)
    for i in range(5):
        nk = torch.randn(1, 2, 1, 128, generator=g)
        nv = torch.randn(1, 2, 1, 128, generator=g)
        cache.append(nk, nv)
        out[f"append_k{i}"] = nk.numpy()
        out[f"append_v{i}"] = nv.numpy()
    q = torch.randn(1, 2, 3, 128, generator=g)
    sc = cache.attention_scores(q)
    w = torch.softmax(sc, dim=-1)
    o = cache.attend(w)
    out.update({"k": k.numpy(), "v": v.numpy(), "q": q.numpy(), "scores": sc.numpy(), "out": o.numpy(),
                "Pi": cache.key_quantizer.mse_quantizer.Pi.numpy(), "S": cache.key_quantizer.S.numpy(),
                "seq_len": np.array(cache.get_seq_length()),
                "memory": np.array([cache.memory_bytes()[n] for n in ("quantized_keys", "quantized_values", "buffer", "total")])})
    np.savez_compressed(os.path.join(HERE, "kv_cache_object.npz"), **out)
    print("kv_cache_object:", len(out), "arrays")


if __name__ == "__main__":
    torch.manual_seed(0)
    steps = {"config1": config1, "key_cases": key_cases, "key_cases_wide": key_cases_wide, "packing": packing,
             "values": values, "codebooks_d256": codebooks_d256, "hybrid": hybrid, "capture_trace": capture_trace,
             "kv_cache_object": kv_cache_object}
    # python tests/golden/make_fixtures.py /root/reference [step ...]   (no step names = all of them)
    for name in (sys.argv[2:] or list(steps)):
        steps[name]()
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))
