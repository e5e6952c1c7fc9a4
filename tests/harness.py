"""The layer arithmetic around the kernels, restated once and run on two back ends.

The reference's `inference/model.py` glues the kernels together with plain int64 tensor ops (scale
ladders, the SiLU gate product, softmax scale 94/695, the causal mask, gate routing, residual adds).
This module restates that glue (file:line cited per function) over a tiny back-end interface so that the
same code runs on the GPU (the `kernel` module + torch) and on the CPU oracle (+ numpy); the tests
compare the two bit for bit.  Nothing here is product code.
"""
import numpy as np


class CpuBackend:
    """numpy arrays + the CPU oracle"""

    def __init__(self, oracle):
        self.o = oracle
        self.lut19 = oracle.softmax_init_q19()
        self.lut23 = oracle.silu_init_q23()

    def linear(self, x, w, shift):
        return self.o.int64_bmm_broadcast(x, w, 1, 1, shift)

    def silu(self, x):
        return self.o.silu_q23(x, self.lut23)

    def sigmoid(self, x):
        return self.o.sigmoid_q23(x, self.lut23)

    def softmax(self, x):
        return self.o.softmax_q19(x, self.lut19)[0]

    def rmsnorm(self, x2d, w, dim):
        return self.o.RMS_Norm_int64(x2d, w, 1, dim)[0]

    def rmsnorm_with_statistic(self, x2d, w, dim):
        """(C, the 500-row statistic buffer the reference returns whole: inference/kernel.py:525, 550)"""
        C, r = self.o.RMS_Norm_int64(x2d, w, 1, dim)
        if not hasattr(self, "rms500"):
            self.rms500 = np.zeros((500,), np.int64)
        self.rms500[:r.shape[0]] = r
        return C, self.rms500

    # ---- witness dump (inference/model.py:94-102: raw C-order bytes); off unless `out` names a directory
    out = None

    def save(self, name, t):
        if self.out is None:
            return
        import os
        path = os.path.join(self.out, name)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "wb") as f:
            f.write(np.ascontiguousarray(self.to_host(t)).tobytes(order="C"))

    def flush(self):
        pass

    def weight_bits(self, w):
        """int32 weights are dumped as their uint32 view (model.py:779): the same bytes"""
        return w

    def residual_rmsnorm(self, x2d, y2d, k, w, dim):
        """(x + y * 2^k, its norm): inference/model.py:1465-1468 op by op"""
        x2d = x2d + y2d * (1 << k)
        return x2d, self.rmsnorm(x2d, w, dim)

    def softmax_scores(self, s1, s2, mask):
        """(scores, probabilities): inference/model.py:896-915 as the reference writes it, op by op"""
        scores = (s1 + s2) * 94 // 695           # floor division (model.py:897)
        if mask is not None:
            scores = scores + mask[:, None, :]   # mask.unsqueeze(1) (model.py:905)
        return scores, self.softmax(scores)

    def silu_mul(self, r1, r2):
        return (self.silu(r1) * r2) >> 23        # model.py:1048 uses // 2^23, :1280 uses >> 23: the same floor

    def silu_mul_keep(self, r1, r2):
        """(SiLU values, gate product): the reference dumps the former (model.py:1042, 1274)"""
        s1 = self.silu(r1)
        return s1, (s1 * r2) >> 23

    def rope(self, x, table):
        return self.o.complex_int64_mul_broadcast(x, table)

    def einsum(self, name, a, b, shift):
        return getattr(self.o, name)(np.ascontiguousarray(a), np.ascontiguousarray(b), shift)

    def causal_mask(self, S, T):
        return np.triu(np.full((S, T), -(64 << 36), np.int64), 1)

    def to_host(self, x):
        return np.asarray(x)

    def from_host(self, x):
        return np.ascontiguousarray(x)

    def zeros_like(self, x):
        return np.zeros_like(x)

    def index_add_rows(self, y, idx, v):
        np.add.at(y, idx, v)
        return y


class GpuBackend:
    """torch CUDA tensors + the HIP library through `kernel`"""

    def __init__(self, kernel):
        import torch
        self.t = torch
        self.k = kernel
        kernel.softmax_init_q19()
        kernel.silu_init_q23()

    def linear(self, x, w, shift):
        return self.k.int64_bmm_broadcast(x.contiguous(), w, 1, 1, shift)

    def silu(self, x):
        out = self.t.empty_like(x)
        self.k.silu_q23(x.contiguous(), out)
        return out

    def sigmoid(self, x):
        out = self.t.empty_like(x)
        self.k.sigmoid_q23(x.contiguous(), out)
        return out

    def softmax(self, x):
        out = self.t.empty_like(x)
        self.k.softmax_q19(x.contiguous(), out)
        return out

    def rmsnorm(self, x2d, w, dim):
        return self.k.RMS_Norm_int64(x2d.contiguous(), w, 1, dim)[0]

    def rmsnorm_with_statistic(self, x2d, w, dim):
        return self.k.RMS_Norm_int64(x2d.contiguous(), w, 1, dim)          # (C, the 500-row host buffer)

    softmax_scores = CpuBackend.softmax_scores   # the same op-by-op chain, on torch tensors
    silu_mul = CpuBackend.silu_mul
    silu_mul_keep = CpuBackend.silu_mul_keep
    residual_rmsnorm = CpuBackend.residual_rmsnorm
    out = None

    def save(self, name, t):
        """the reference's saveTensor as the reference calls it: a synchronous copy to the host, then the file"""
        if self.out is None:
            return
        import os
        path = os.path.join(self.out, name)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        if isinstance(t, np.ndarray):
            t = self.t.from_numpy(np.ascontiguousarray(t))
        t = t.detach().cpu().contiguous()
        with open(path, "wb") as f:
            f.write(t.numpy().tobytes(order="C"))

    def flush(self):
        pass

    def weight_bits(self, w):
        return w

    def rope(self, x, table):
        return self.k.complex_int64_mul_broadcast(x.contiguous(), table.contiguous())

    def einsum(self, name, a, b, shift):
        return getattr(self.k, name)(a.contiguous(), b.contiguous(), shift)

    def causal_mask(self, S, T):
        return self.t.full((S, T), -(64 << 36), dtype=self.t.int64, device="cuda").triu_(1)

    def to_host(self, x):
        return x.cpu().numpy()

    def from_host(self, x):
        return self.t.from_numpy(np.ascontiguousarray(x)).cuda()

    def zeros_like(self, x):
        return self.t.zeros_like(x)

    def index_add_rows(self, y, idx, v):
        y.index_add_(0, idx, v)
        return y


class FusedGpuBackend(GpuBackend):
    """GpuBackend that takes the library's fused entry points where the reference chains tensor ops around a kernel"""

    def softmax_scores(self, s1, s2, mask):
        scores, p = self.t.empty_like(s1), self.t.empty_like(s1)
        self.k.softmax_q19_scores(s1.contiguous(), s2.contiguous(), None if mask is None else mask.contiguous(), p, scores)
        return scores, p

    def silu_mul(self, r1, r2):
        out = self.t.empty_like(r1)
        self.k.silu_mul_q23(r1.contiguous(), r2.contiguous(), out)
        return out

    def silu_mul_keep(self, r1, r2):
        s1, out = self.t.empty_like(r1), self.t.empty_like(r1)
        self.k.silu_mul_q23(r1.contiguous(), r2.contiguous(), out, S=s1)
        return s1, out

    def residual_rmsnorm(self, x2d, y2d, k, w, dim):
        xn, c, _ = self.k.RMS_Norm_residual_int64(x2d.contiguous(), y2d.contiguous(), k, w, 1, dim)
        return xn, c

    def rmsnorm_with_statistic(self, x2d, w, dim):
        # the statistic stays on the device (no wait); the dump writer copies it behind the kernels
        return self.k.RMS_Norm_int64(x2d.contiguous(), w, 1, dim, host_rms=False)

    def save(self, name, t):
        """through the library's dump writer: device tensors are handed over as they are (no .cpu())"""
        if self.out is None:
            return
        import os
        path = os.path.join(self.out, name)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        if isinstance(t, np.ndarray):
            t = self.t.from_numpy(np.ascontiguousarray(t))
        self.k.saveTensor(path, t)

    def flush(self):
        self.k.dump_flush()

    def sigmoid_route(self, logits, bias_host, cfg):
        """sigmoid and routing in one launch: returns the sigmoid scores, keeps the routing for route()"""
        bias = self.t.from_numpy(bias_host.astype(np.int32)).cuda()
        raw = self.t.empty((logits.shape[1], cfg["topk"]), dtype=self.t.int64, device="cuda")
        sc, w, idx = self.k.gate_sigmoid_route(logits[0].contiguous(), bias, cfg["groups"], cfg["topk_groups"], cfg["topk"],
                                               raw_weights=raw)
        self._routed = (w, idx, raw)
        return sc[None]

    def route(self, scores, bias_host, cfg):
        if getattr(self, "_routed", None) is not None:
            w, idx, raw = self._routed
            self._routed = None
        else:
            bias = self.t.from_numpy(bias_host.astype(np.int32)).cuda()
            raw = self.t.empty((scores.shape[0], cfg["topk"]), dtype=self.t.int64, device="cuda")
            w, idx = self.k.gate_route(scores.contiguous(), bias, cfg["groups"], cfg["topk_groups"], cfg["topk"], raw_weights=raw)
        self.last_route = (w, idx)
        self.last_raw_weights = raw
        return w.cpu().numpy(), idx.cpu().numpy()

    def routed_experts(self, x, P, cfg):
        """every routed expert in one go, from the routing result that is still on the device"""
        w, idx = self.last_route
        key = id(P["w1"])
        if getattr(self, "_tables_for", None) != key:
            self._tables = tuple(self.k.pointer_table(P[n]) for n in ("w1", "w3", "w2"))
            self._tables_for = key
        t1, t3, t2 = self._tables
        b32 = P["w1"][0].dtype == self.t.int32
        dump = None
        if self.out is not None and getattr(self, "layer_dir", None):
            import os
            dump = os.path.join(self.out, self.layer_dir)
        return self.k.moe_experts(x[0].contiguous(), w, idx, t1, t3, t2, b32, cfg["inter"], cfg["c13"], cfg["c2"], dump_dir=dump)


class CheckedGpuBackend(GpuBackend):
    """GpuBackend that checks every kernel call against the CPU oracle on the call's ACTUAL inputs: completely
    when the call is small, on a seeded sample of output rows/columns/heads otherwise.  A chain run through it
    is verified link by link at sizes where a whole-chain CPU run would take hours."""

    def __init__(self, kernel, cpu, seed=0, full_limit=1 << 27):
        super().__init__(kernel)
        self.cpu = cpu
        self.rng = np.random.default_rng(seed)
        self.full_limit = full_limit          # multiply-adds (or elements) up to which a call is checked in full
        self.checked = {}

    def _count(self, what, n):
        self.checked[what] = self.checked.get(what, 0) + int(n)

    def _pick(self, n, k):
        if n <= k:
            return np.arange(n)
        return np.unique(np.concatenate([[0, n - 1], self.rng.integers(0, n, k - 2)]))

    def _dev(self, idx):
        return self.t.from_numpy(np.asarray(idx, dtype=np.int64)).cuda()

    def linear(self, x, w, shift):
        C, R = super().linear(x, w, shift)
        M, K, N = x.shape[1], x.shape[2], w.shape[0]
        rows = np.arange(M) if M * N * K <= self.full_limit else self._pick(M, 3)
        cols = np.arange(N) if M * N * K <= self.full_limit else self._pick(N, 48)
        xr, wc = x[:, self._dev(rows)], w[self._dev(cols)]
        Ce, Re = self.cpu.linear(xr.cpu().numpy(), wc.cpu().numpy(), shift)
        sub = lambda t: t[:, self._dev(rows)][:, :, self._dev(cols)].cpu().numpy()
        assert np.array_equal(sub(C), Ce), "linear: quotient differs from the oracle"
        assert np.array_equal(sub(R), Re), "linear: remainder differs from the oracle"
        self._count("linear", rows.size * cols.size)
        return C, R

    def _rowwise(self, what, gpu_fn, cpu_fn, x):
        out = gpu_fn(x)
        flat_in, flat_out = x.reshape(-1, x.shape[-1]), out.reshape(-1, x.shape[-1])
        rows = np.arange(flat_in.shape[0]) if x.numel() <= self.full_limit else self._pick(flat_in.shape[0], 4096)
        got = flat_out[self._dev(rows)].cpu().numpy()
        want = cpu_fn(np.ascontiguousarray(flat_in[self._dev(rows)].cpu().numpy()))
        assert np.array_equal(got, want), what + " differs from the oracle"
        self._count(what, got.size)
        return out

    def silu(self, x):
        return self._rowwise("silu", super().silu, self.cpu.silu, x)

    def sigmoid(self, x):
        return self._rowwise("sigmoid", super().sigmoid, self.cpu.sigmoid, x)

    def softmax(self, x):
        cpu_fn = lambda rows: self.cpu.softmax(rows[None, None])[0, 0]
        return self._rowwise("softmax", super().softmax, cpu_fn, x)

    def rmsnorm(self, x2d, w, dim):
        out = super().rmsnorm(x2d, w, dim)
        want = self.cpu.rmsnorm(x2d.cpu().numpy(), w.cpu().numpy(), dim)
        assert np.array_equal(out.cpu().numpy(), want), "rmsnorm differs from the oracle"
        self._count("rmsnorm", want.size)
        return out

    def rmsnorm_with_statistic(self, x2d, w, dim):
        return self.rmsnorm(x2d, w, dim), self.k.rms

    def rope(self, x, table):
        out = super().rope(x, table)
        want = self.cpu.rope(np.ascontiguousarray(x.cpu().numpy()), np.ascontiguousarray(table.cpu().numpy()))
        assert np.array_equal(out.cpu().numpy(), want), "rope differs from the oracle"
        self._count("rope", want.size)
        return out

    def einsum(self, name, a, b, shift):
        out = super().einsum(name, a, b, shift)
        S, H = a.shape[1], a.shape[2]
        macs = out.numel() * a.shape[3]
        ss = np.arange(S) if macs <= self.full_limit else self._pick(S, 3)
        hs = np.arange(H) if macs <= self.full_limit else self._pick(H, 4)
        asub = a[:, self._dev(ss)][:, :, self._dev(hs)].contiguous().cpu().numpy()
        per_head = name in ("einsum_bshd_hdc_bshc", "einsum_bshc_hdc_bshd")          # b is [H, D, C]
        bsub = (b[self._dev(hs)] if per_head else b).contiguous().cpu().numpy()
        want = self.cpu.einsum(name, asub, bsub, shift)
        got = out[:, self._dev(ss)][:, :, self._dev(hs)].cpu().numpy()
        assert np.array_equal(got, want), name + " differs from the oracle"
        self._count(name, got.size)
        return out


def expert_ffn(be, x, w1, w2, w3, c13, c2, dump=None):
    """gate/up GEMMs, SiLU gate, down GEMM: MLP_int.forward / Expert_int.forward
    (inference/model.py:1018-1049, 1247-1281).  x [1,M,dim] Q23 activations."""
    r1, _ = be.linear(x, w1, c13)
    r2, _ = be.linear(x, w3, c13)
    if dump:                                  # file names of model.py:1037-1042 (shared expert) / :1269-1274 (routed)
        s1, h = be.silu_mul_keep(r1, r2)
        be.save(dump + "_x.bin", r1)
        be.save(dump + "_y.bin", s1)
    else:
        h = be.silu_mul(r1, r2)
    y, _ = be.linear(h, w2, c2)
    return y


def attention_scores_softmax_pv(be, q_nope, q_pe, kv_cache, pe_cache, causal=True, layer_dir=None):
    """scores = ((q_nope.kv + 11)>>23 + (q_pe.pe + 10)>>21) * 94 // 695 + mask; softmax_q19; P.V >> 23
    (inference/model.py:884-936).  q_nope [1,S,H,C], q_pe [1,S,H,R], kv_cache [1,T,C], pe_cache [1,T,R]."""
    s1 = be.einsum("einsum_bshc_btc_bsht", q_nope, kv_cache, 23)
    s2 = be.einsum("einsum_bshc_btc_bsht", q_pe, pe_cache, 21)
    scores, p = be.softmax_scores(s1, s2, be.causal_mask(s1.shape[1], s1.shape[3]) if causal else None)
    if layer_dir:
        be.save(layer_dir + "/scores_softmax_x.bin", scores)            # model.py:913, 918
        be.save(layer_dir + "/scores_softmax_y.bin", p)
    out = be.einsum("einsum_bsht_btc_bshc", p, kv_cache, 23)
    return scores, p, out


def mla(be, x, P, freqs, cfg, layer_dir=None):
    """MLA.forward in absorb mode at start_pos = 0 (inference/model.py:747-957).  x [1,S,dim]."""
    S, H = x.shape[1], cfg["heads"]
    cq, ckv = cfg.get("c_q", 30), cfg.get("c_kv", 29)           # the model's scales (model.py:772-833); tests may pick others
    q_down, q_down_rem = be.linear(x, P["wq_a"], cq)
    q_normed, q_rms = be.rmsnorm_with_statistic(q_down[0], P["q_norm"], cfg["q_lora"])
    q_normed = q_normed[None]
    if layer_dir:                             # model.py:776-793
        be.save(layer_dir + "/wq_a_x.bin", x)
        be.save(layer_dir + "/wq_a_w.bin", be.weight_bits(P["wq_a"]))
        be.save(layer_dir + "/wq_a_y.bin", q_down)
        be.save(layer_dir + "/q_norm_r.bin", q_down_rem)
        be.save(layer_dir + "/q_norm_x.bin", q_down)
        be.save(layer_dir + "/q_norm_weight.bin", be.weight_bits(P["q_norm"]))
        be.save(layer_dir + "/q_norm_rms.bin", q_rms)
        be.save(layer_dir + "/q_norm_y.bin", q_normed)
    q_nope, _ = be.linear(q_normed, P["wq_b1"], cq)
    q_pe, _ = be.linear(q_normed, P["wq_b2"], cq)
    q_nope = q_nope.reshape(1, S, H, cfg["nope"])
    if layer_dir:                             # model.py:813-819 (q_pe_y.bin really receives the q_norm weights there)
        be.save(layer_dir + "/q_pe_x.bin", q_pe.reshape(1, S, H, cfg["rope"]))
        be.save("freqs_cis.bin", freqs)
        be.save(layer_dir + "/q_pe_y.bin", be.weight_bits(P["q_norm"]))
    q_pe = q_pe.reshape(1, S, H, cfg["rope"] // 2, 2)
    q_pe = be.rope(q_pe, freqs).reshape(1, S, H, cfg["rope"])
    kv, kv_rem = be.linear(x, P["wkv_a1"], ckv)
    if layer_dir:                             # model.py:830-833
        be.save(layer_dir + "/wkv_a1_x.bin", x)
        be.save(layer_dir + "/wkv_a1_w.bin", be.weight_bits(P["wkv_a1"]))
        be.save(layer_dir + "/wkv_a1_y.bin", kv)
        be.save(layer_dir + "/wkv_a1_r.bin", kv_rem)
    k_pe, _ = be.linear(x, P["wkv_a2"], ckv)
    k_pe = be.rope(k_pe.reshape(1, S, 1, cfg["rope"] // 2, 2), freqs).reshape(1, S, cfg["rope"])
    q_abs = be.einsum("einsum_bshd_hdc_bshc", q_nope, P["wkv_b_1"], cfg["wkv_b_1_scale"])
    kv_normed = be.rmsnorm(kv[0], P["kv_norm"], cfg["kv_lora"])[None]
    _, _, o = attention_scores_softmax_pv(be, q_abs, q_pe, kv_normed, k_pe, layer_dir=layer_dir)
    o = be.einsum("einsum_bshc_hdc_bshd", o, P["wkv_b_2"], cfg["wkv_b_2_scale"])
    y, _ = be.linear(o.reshape(1, S, H * cfg["v"]), P["wo"], cfg["wo_scale"])
    return y


def gate_scores(be, x, P, cfg, layer_dir=None):
    """the kernel part of Gate.forward: linear at the gate's scale, then sigmoid_q23 (model.py:1116-1135)"""
    s, s_rem = be.linear(x, P["gate"], cfg["gate_scale"])
    c = be.sigmoid_route(s, P["gate_bias_host"], cfg) if hasattr(be, "sigmoid_route") else be.sigmoid(s)
    if layer_dir:                             # model.py:1132-1138, 1151-1152
        be.save(layer_dir + "/sigmoid_gate_x.bin", s)
        be.save(layer_dir + "/sigmoid_gate_r.bin", s_rem)
        be.save(layer_dir + "/sigmoid_gate_y.bin", c)
        be.save(layer_dir + "/gate_original_scores.bin", c[0])
        be.save(layer_dir + "/gate_bias.bin", P["gate_bias_host"].astype(np.int32))
    return c[0]


def route(scores_host, bias, cfg):
    """the tensor-op part of Gate.forward (model.py:1160-1208) on the host, with exact integers; returns
    (weights [T,topk], indices [T,topk]).  Ties are broken by lowest index, as a stable sort does."""
    T, E = scores_host.shape
    orig = scores_host
    sc = scores_host + bias[None, :]
    g = cfg["groups"]
    grp = sc.reshape(T, g, E // g)
    top2 = -np.sort(-grp, axis=-1)[..., :2].sum(-1)
    gsel = np.argsort(-top2, axis=-1, kind="stable")[:, :cfg["topk_groups"]]
    keep = np.zeros((T, g), bool)
    np.put_along_axis(keep, gsel, True, axis=1)
    sc = np.where(np.repeat(keep, E // g, axis=1), sc, -(1 << 42))
    idx = np.argsort(-sc, axis=-1, kind="stable")[:, :cfg["topk"]]
    w = np.take_along_axis(orig, idx, axis=1)
    w = (w * (1 << 23)) // w.sum(-1, keepdims=True)
    w = w * 5 // 2
    return w, idx


def moe(be, x, P, cfg, layer_dir=None):
    """MoE.forward (inference/model.py:1325-1383): shared expert + top-k routed experts, weights Q23"""
    T = x.shape[1]
    shared = layer_dir + "/mlp_silu" if layer_dir else None
    z = expert_ffn(be, x, P["sw1"], P["sw2"], P["sw3"], cfg["c13"], cfg["c2"], dump=shared)      # model.py:1346
    sc = gate_scores(be, x, P, cfg, layer_dir)
    if hasattr(be, "route"):
        w_host, idx_host = be.route(sc, P["gate_bias_host"], cfg)
        raw = be.last_raw_weights
    else:
        sc_host = be.to_host(sc)
        w_host, idx_host = route(sc_host, P["gate_bias_host"], cfg)
        raw = np.take_along_axis(sc_host, idx_host, axis=1)
    if layer_dir:                             # model.py:1196-1197: the winners' unbiased scores, before they are normalised
        be.save(layer_dir + "/gate_indices.bin", idx_host.astype(np.int64) if not hasattr(be, "route") else be.last_route[1])
        be.save(layer_dir + "/gate_weights.bin", raw)
    if hasattr(be, "routed_experts"):
        be.layer_dir = layer_dir
        y = be.routed_experts(x, P, cfg)
        return y[None] + z, idx_host
    y = be.zeros_like(x[0])
    for e in range(cfg["experts"]):
        tok, slot = np.nonzero(idx_host == e)
        if tok.size == 0:
            continue
        xe = x[0][be.from_host(tok)][None]
        ye = expert_ffn(be, xe, P["w1"][e], P["w2"][e], P["w3"][e], cfg["c13"], cfg["c2"],
                        dump=layer_dir + "/expert_%d_silu" % e if layer_dir else None)[0]
        we = be.from_host(w_host[tok, slot].astype(np.int64))[:, None]
        y = be.index_add_rows(y, be.from_host(tok), (ye * we) // (1 << 23))      # model.py:1379
    return y[None] + z, idx_host


def decoder_layer(be, x, P, freqs, cfg, layer_dir=None):
    """Block.forward for a MoE layer (inference/model.py:1430-1475): x Q31 residual stream [1,S,dim].  With `layer_dir`
    (e.g. "pos_0/layer_3") and a back end whose `out` names a directory, the witness files the reference writes for
    the layer are written under it, with the reference's names and bytes."""
    a, a_rms = be.rmsnorm_with_statistic(x[0], P["attn_norm"], cfg["dim"])
    a = a[None]
    if layer_dir:                             # model.py:1455-1458
        be.save(layer_dir + "/attn_norm_x.bin", x)
        be.save(layer_dir + "/attn_norm_weight.bin", be.weight_bits(P["attn_norm"]))
        be.save(layer_dir + "/attn_norm_y.bin", a)
        be.save(layer_dir + "/attn_norm_rms.bin", a_rms)
    x, f = be.residual_rmsnorm(x[0], mla(be, a, P, freqs, cfg, layer_dir)[0], 12, P["ffn_norm"], cfg["dim"])   # model.py:1465-1468
    x, f = x[None], f[None]
    y, idx = moe(be, f, P, cfg, layer_dir)
    be.flush()
    return x + y * (1 << 8), idx                                 # model.py:1472
