import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "strix.rs_amd")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def _load_by_path(name, path, search=None):
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=search)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    """The product package (directory name has a dot, so it is loaded by path)."""
    return _load_by_path("strix_rs_amd", os.path.join(PKG_DIR, "__init__.py"), [PKG_DIR])


@pytest.fixture(scope="session")
def synth():
    return _load_by_path("strix_rs_amd_synth", os.path.join(PKG_DIR, "synth.py"))


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    return _load_by_path("strix_oracle", os.path.join(ROOT, "oracle", "strix_oracle.py"))


@pytest.fixture(scope="session")
def accel(pkg):
    """One context for the whole GPU session; fails loudly without the built library or a GPU."""
    a = pkg.Mi355WeightAccel(0)
    yield a
    a.close()


def rel_err(got, ref):
    """max|got-ref| / max|ref|: the reference's normalisation (strix-backend-rocm/src/lib.rs:217-222)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


@pytest.fixture(scope="session")
def relerr():
    return rel_err


GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


@pytest.fixture(scope="session")
def golden():
    def load(name):
        return np.load(os.path.join(GOLDEN_DIR, name), allow_pickle=False)
    return load


EXPERT_BLOCK = {8: (32, 34), 14: (256, 210)}   # ggml type -> (elements, bytes) per block


def expert_rows(raw, ty, e, rows, in_dim):
    """Raw bytes of expert e out of a stacked expert tensor [ne][rows][in_dim/QK blocks]."""
    be, bb = EXPERT_BLOCK[ty]
    per = rows * (in_dim // be) * bb
    return np.asarray(raw, np.uint8).reshape(-1)[e * per:(e + 1) * per]


def moe_layer_stagewise(accel, orc, layer, ty, gate, up, down, ne, hidden, eff, xs, plan, slot_tok, wslot, groups=None, tol=1e-5):
    """Stage-by-stage parity of the grouped (prefill) MoE path, the way the decode path is checked:
    gate/up of every slot against the oracle's Q8 matmul of the slot's expert on the slot's token;
    the re-quantised silu(g)*u bit-exact on the device's own g, u; the down GEMM from the device's own
    quants; the weighted combine in ascending slot order.  `groups`: indices of the plan entries to
    check against the oracle (all when None); the combine is always checked for every token."""
    m = xs.shape[0]
    y, gu, aq, ad, dy = accel.moe_layer_stages(layer, xs, m, plan, slot_tok, wslot, eff)
    xq, xd, _ = orc.actquant(xs, hidden)
    worst = {"gate_up": 0.0, "down": 0.0, "combine": 0.0}
    for gi in (range(len(plan)) if groups is None else groups):
        e, off, cnt = (int(v) for v in plan[gi])
        toks = slot_tok[off:off + cnt]
        for z, w3 in enumerate((gate, up)):
            ref = orc.matmul_q8(ty, expert_rows(w3, ty, e, eff, hidden), hidden, eff, xq[toks], xd[toks])
            worst["gate_up"] = max(worst["gate_up"], rel_err(gu[off:off + cnt, z], ref))
        a = orc.act_produce(2, gu[off:off + cnt, 0].reshape(-1), gu[off:off + cnt, 1].reshape(-1)).reshape(cnt, eff)
        q2, d2, _ = orc.actquant(a, eff)
        assert np.array_equal(aq[off:off + cnt], q2), f"group {gi}: quantised silu(g)*u differs"
        assert np.array_equal(ad[off:off + cnt].view(np.uint32), d2.view(np.uint32)), f"group {gi}: block scales differ"
        ref = orc.matmul_q8(ty, expert_rows(down, ty, e, hidden, eff), eff, hidden, aq[off:off + cnt], ad[off:off + cnt])
        worst["down"] = max(worst["down"], rel_err(dy[off:off + cnt], ref))
    want = np.zeros((m, hidden), np.float32)
    for s in range(slot_tok.size):          # ascending slot index per token, fp32 multiply then add
        want[slot_tok[s]] += np.float32(wslot[s]) * dy[s]
    worst["combine"] = rel_err(y, want)
    assert worst["gate_up"] <= tol and worst["down"] <= tol and worst["combine"] <= tol, worst
    return y, worst


@pytest.fixture(scope="session")
def moe_stagewise():
    return moe_layer_stagewise
