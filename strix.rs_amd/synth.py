"""Seeded synthetic tensors in the GGUF block formats of the quantized-matmul path.

Distributions follow the benchmark configurations: f16 block scales uniform in
a given range, uniformly random quants, N(0,1) activations, Zipf(1.1) expert
popularity for MoE routing.  Layout is the raw GGUF one the upload entry points
take: row-major over out_dim rows, each row in_dim/QK consecutive blocks.
"""
import numpy as np

Q4_0, Q8_0, Q6_K = 2, 8, 14
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q6_K: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q6_K: 210}


def _f16_scales(rng, n, lo, hi):
    return rng.uniform(lo, hi, n).astype(np.float32).astype(np.float16).view(np.uint16)


def make_q4_0(out_dim, in_dim, seed, dlo=0.001, dhi=0.02):
    """Q4_0: [f16 d][16 nibble bytes], value (q-8)*d."""
    rng = np.random.default_rng(seed)
    nblk = out_dim * (in_dim // 32)
    raw = np.empty((nblk, 18), np.uint8)
    raw[:, 0:2] = _f16_scales(rng, nblk, dlo, dhi).view(np.uint8).reshape(nblk, 2)
    raw[:, 2:] = rng.integers(0, 256, (nblk, 16), dtype=np.uint8)
    return raw.reshape(-1)


def make_q8_0(out_dim, in_dim, seed, dlo=0.001, dhi=0.02):
    """Q8_0: [f16 d][32 x i8 in -127..127]."""
    rng = np.random.default_rng(seed)
    nblk = out_dim * (in_dim // 32)
    raw = np.empty((nblk, 34), np.uint8)
    raw[:, 0:2] = _f16_scales(rng, nblk, dlo, dhi).view(np.uint8).reshape(nblk, 2)
    raw[:, 2:] = rng.integers(-127, 128, (nblk, 32), dtype=np.int8).view(np.uint8)
    return raw.reshape(-1)


def make_q6_k(out_dim, in_dim, seed, dlo=1e-4, dhi=2e-3):
    """Q6_K: [128 ql][64 qh][16 x i8 sub-scales in -64..63][f16 d]."""
    rng = np.random.default_rng(seed)
    nsb = out_dim * (in_dim // 256)
    raw = np.empty((nsb, 210), np.uint8)
    raw[:, 0:192] = rng.integers(0, 256, (nsb, 192), dtype=np.uint8)
    raw[:, 192:208] = rng.integers(-64, 64, (nsb, 16), dtype=np.int8).view(np.uint8)
    raw[:, 208:210] = _f16_scales(rng, nsb, dlo, dhi).view(np.uint8).reshape(nsb, 2)
    return raw.reshape(-1)


def make_weight(ty, out_dim, in_dim, seed):
    return {Q4_0: make_q4_0, Q8_0: make_q8_0, Q6_K: make_q6_k}[ty](out_dim, in_dim, seed)


def make_acts(m, in_dim, seed):
    """fp32 activations ~ N(0,1), shape [m, in_dim]."""
    return np.random.default_rng(seed).standard_normal((m, in_dim), dtype=np.float32)


def make_moe_q8(ne, hidden, eff, seed):
    """Expert tensors as GGUF stores them: gate/up [ne][eff][hidden/32 blocks], down [ne][hidden][eff/32]."""
    gate = make_q8_0(ne * eff, hidden, seed)
    up = make_q8_0(ne * eff, hidden, seed + 1)
    down = make_q8_0(ne * hidden, eff, seed + 2)
    return gate, up, down


def make_moe_q6(ne, hidden, eff, seed):
    """The same tensors as Q6_K superblocks (hidden and eff multiples of 256)."""
    gate = make_q6_k(ne * eff, hidden, seed)
    up = make_q6_k(ne * eff, hidden, seed + 1)
    down = make_q6_k(ne * hidden, eff, seed + 2)
    return gate, up, down


def zipf_routing(m, ne, k, seed, s=1.1):
    """Per token: k distinct experts drawn without replacement with Zipf(s) popularity,
    weights = renormalised softmax of N(0,1) logits.  Returns ids[m][k] i32, w[m][k] f32."""
    rng = np.random.default_rng(seed)
    p = 1.0 / np.arange(1, ne + 1, dtype=np.float64) ** s
    p /= p.sum()
    perm = rng.permutation(ne)  # which expert is the popular one is arbitrary
    ids = np.empty((m, k), np.int32)
    for t in range(m):
        ids[t] = perm[rng.choice(ne, size=k, replace=False, p=p)]
    logits = rng.standard_normal((m, k)).astype(np.float32)
    e = np.exp(logits - logits.max(axis=1, keepdims=True))
    w = (e / e.sum(axis=1, keepdims=True)).astype(np.float32)
    return ids, w


def group_by_expert(ids, w, ne):
    """(token, slot) pairs grouped by expert, as the CPU forward builds them before
    calling the whole-layer MoE entry point: plan rows (expert, slot_off, count),
    slot_tok[slots], wslot[slots]."""
    m, k = ids.shape
    plan, slot_tok, wslot = [], [], []
    for e in range(ne):
        toks, slots = np.nonzero(ids == e)
        if toks.size == 0:
            continue
        plan.append((e, len(slot_tok), int(toks.size)))
        slot_tok.extend(int(t) for t in toks)
        wslot.extend(float(w[t, s]) for t, s in zip(toks, slots))
    return (np.asarray(plan, np.int64).reshape(-1, 3), np.asarray(slot_tok, np.int32),
            np.asarray(wslot, np.float32))
