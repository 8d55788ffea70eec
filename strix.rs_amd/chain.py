"""The FFN half of a decoder stack as a sequence of resident, device-routed calls: what an orchestrator captures once
as a HIP graph and replays per token (the reference's captured token, crates/strix-backend-rocm/src/decode.rs:3053-3203,
and its per-layer launch sequence, decode.rs:1136-1180: router logits -> topk_router -> moe_launches).

Per layer, four calls / five launches:
    1. smx_ffn_gate_up_dev     rmsnorm + quantiser + gate and up GEMVs + SwiGLU product   x -> h[ffn]
    2. smx_gemv_dev            quantiser + down GEMV                                      h -> d[hidden]
    3. smx_gemv_dev            router logits GEMV                                         d -> logits[ne]
    4. smx_moe_ffn_logits_dev  softmax + top-k in the prologue of the k routed experts' gate/up launch, then their down
                               launch                                                     d, logits -> y[hidden] (+ ids[k], w[k])
(route="call": the router as smx_moe_router_dev, route="launches": as smx_gemv_dev + smx_moe_route_dev, each followed by
smx_moe_ffn_routed_dev: six launches, same bits.)
Attention, RoPE and the KV cache are outside this path.  The benchmark (bench.py) and the parity test
(tests/test_gpu_chain.py) both run this class, so what is measured is what is checked.
"""


class FfnMoeChain:
    """keys(l) -> (gate, up, down, router) weight keys of layer l; moe_layer(l) -> resident MoE layer index.

    keep_stages: every layer gets buffers of its own for h, d, logits, ids, w and y, so that a test can read each stage back;
    otherwise the layers share one set (what a decode loop does)."""

    def __init__(self, acc, layers, hidden, ffn, ne, k, keys, moe_layer, norm_w_dev, eps=1e-6, keep_stages=False,
                 route="in_launch"):
        self.acc, self.layers, self.hidden, self.ffn, self.ne, self.k = acc, layers, hidden, ffn, ne, k
        self.keys, self.moe_layer, self.norm_w_dev, self.eps = keys, moe_layer, norm_w_dev, eps
        assert route in ("in_launch", "call", "launches")
        self.route = route
        self._bufs = []
        nsets = layers if keep_stages else 1
        self.stage = []
        for _ in range(nsets):
            b = {"h": self._alloc(ffn * 4), "d": self._alloc(hidden * 4), "logits": self._alloc(ne * 4),
                 "ids": self._alloc(k * 4), "w": self._alloc(k * 4)}
            self.stage.append(b)
        # layer outputs alternate between two buffers (a layer reads the previous layer's output); with keep_stages each its own
        self.y = [self._alloc(hidden * 4) for _ in range(layers if keep_stages else 2)]

    def _alloc(self, nbytes):
        p = self.acc.dev_alloc(nbytes)
        self._bufs.append(p)
        return p

    def buffers(self, l):
        """(stage buffers, output buffer) of layer l."""
        return self.stage[l % len(self.stage)], self.y[l % len(self.y)]

    def enqueue(self, x_dev, layer_offset=0):
        """Enqueue all layers on the context's stream (capturable); returns the device buffer holding the last layer's output.
        layer_offset: added to the layer index when naming weights (rotating weight sets of a benchmark)."""
        acc, cur = self.acc, x_dev
        for l in range(self.layers):
            b, y = self.buffers(l)
            gate, up, down, router = self.keys(l + layer_offset)
            ok = acc.ffn_gate_up_dev(gate, up, 2, cur, b["h"], norm=True, norm_w_dev=self.norm_w_dev, eps=self.eps)
            ok = ok and acc.gemv_dev(down, b["h"], 1, b["d"])
            layer = self.moe_layer(l + layer_offset)
            if self.route == "in_launch":
                ok = ok and acc.gemv_dev(router, b["d"], 1, b["logits"])
                ok = ok and acc.moe_ffn_logits_dev(layer, b["logits"], self.k, b["d"], y, b["ids"], b["w"])
            else:
                if self.route == "call":
                    ok = ok and acc.moe_router_dev(router, b["d"], self.k, b["ids"], b["w"], b["logits"])
                else:
                    ok = ok and acc.gemv_dev(router, b["d"], 1, b["logits"])
                    ok = ok and acc.moe_route_dev(b["logits"], self.ne, self.k, b["ids"], b["w"])
                ok = ok and acc.moe_ffn_routed_dev(layer, b["ids"], b["w"], self.k, b["d"], y)
            if not ok:
                raise RuntimeError(f"layer {l}: a weight of the chain is not resident")
            cur = y
        return cur

    def launches_per_token(self):
        """(when the experts' gate/up launch routes: up to 64 experts, k <= 8, flat-form expert rows)"""
        return self.layers * (5 if self.route == "in_launch" else 6)

    def close(self):
        for p in self._bufs:
            self.acc.dev_free(p)
        self._bufs = []
