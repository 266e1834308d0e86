"""Shared test helpers: seeded synthetic data and error measures."""
from __future__ import annotations

import numpy as np

import oracle


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def normal_bf16(seed: int, shape, std: float = 1.0, mean: float = 0.0) -> np.ndarray:
    return oracle.f32_to_bf16((rng(seed).standard_normal(shape, dtype=np.float32) * std + mean).astype(np.float32))


def make_qweight(seed: int, n: int, k: int, bits: int = 4, group: int = 64, std: float = 0.02) -> oracle.QWeight:
    """W ~ N(0, std^2) in fp32 from PCG64(seed), MLX-affine quantised (bits 4/8) or rounded to bf16 (bits 16)."""
    w = (rng(seed).standard_normal((n, k), dtype=np.float32) * std).astype(np.float32)
    if bits == 16:
        return oracle.dense(oracle.f32_to_bf16(w))
    return oracle.quantize(w, bits, group)


def rel_l2(got_bf16: np.ndarray, ref_f32: np.ndarray) -> float:
    g = oracle.bf16_to_f32(got_bf16).astype(np.float64).ravel()
    r = np.asarray(ref_f32, dtype=np.float64).ravel()
    return float(np.linalg.norm(g - r) / max(np.linalg.norm(r), 1e-30))


def bf16_mismatch(a: np.ndarray, b: np.ndarray):
    """(fraction of elements whose bf16 bits differ, max difference in bf16 ulps of the larger magnitude)."""
    a = np.asarray(a, dtype=np.uint16).ravel()
    b = np.asarray(b, dtype=np.uint16).ravel()
    diff = a != b
    if not diff.any():
        return 0.0, 0.0
    fa, fb = oracle.bf16_to_f32(a).astype(np.float64), oracle.bf16_to_f32(b).astype(np.float64)
    mag = np.maximum(np.abs(fa), np.abs(fb))
    ulp = np.where(mag > 0, 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-38))) - 7), 1e-38)
    return float(diff.mean()), float((np.abs(fa - fb) / ulp).max())


def to_device(fk, W: oracle.QWeight):
    return fk.DeviceWeight(W.w, W.scales, W.biases, W.n, W.k, W.bits, W.group)


# ---------------------------------------------------------------- whole-model oracle
class HostDecoderWeights:
    """A dense decoder's weights built on the HOST with the oracle's copy of the library's
    host-reproducible generator and the oracle's quantiser: the bytes
    `DecoderWeights.random_init(cfg, seed, exact=True, ...)` puts into HBM (same seed sequence)."""

    def __init__(self, cfg, seed: int = 0, std: float = 0.02, embed_seed=None, embed_tau: float = 0.0,
                 with_embedding: bool = True, embed_loud_rows: int = 0, embed_loud_gain: float = 1.0):
        self.cfg = cfg
        self.mats, self.vecs = {}, {}
        self.std = std
        counter = [seed * 100003 + 1]

        def next_seed():
            counter[0] += 1
            return counter[0]

        def matrix(name, n, k):
            sd = next_seed()
            if cfg.bits == 16:
                self.mats[name] = oracle.dense(oracle.synth_fill(n * k, sd, 0.0, std, 4).reshape(n, k))
            else:
                self.mats[name] = oracle.quantize(oracle.synth_fill(n * k, sd, 0.0, std, 3).reshape(n, k), cfg.bits, cfg.group)

        def vector(name, n, mean, sd_):
            self.vecs[name] = oracle.synth_fill(n, next_seed(), mean, sd_, 4)

        es = next_seed()
        self.embed_seed = es if embed_seed is None else embed_seed
        if with_embedding:
            self.set_embedding(self.embed_seed, embed_tau, embed_loud_rows, embed_loud_gain)
        vector("final_norm", cfg.hidden, 1.0, 0.1)
        for l in range(cfg.n_layers):
            p = f"layers.{l}."
            matrix(p + "self_attn.q_proj", cfg.n_q, cfg.hidden)
            matrix(p + "self_attn.k_proj", cfg.n_kvd, cfg.hidden)
            matrix(p + "self_attn.v_proj", cfg.n_kvd, cfg.hidden)
            matrix(p + "self_attn.o_proj", cfg.hidden, cfg.n_q)
            matrix(p + "mlp.gate_proj", cfg.inter, cfg.hidden)
            matrix(p + "mlp.up_proj", cfg.inter, cfg.hidden)
            matrix(p + "mlp.down_proj", cfg.hidden, cfg.inter)
            vector(p + "input_layernorm", cfg.hidden, 1.0, 0.1)
            vector(p + "post_attention_layernorm", cfg.hidden, 1.0, 0.1)
            if cfg.qk_norm:
                vector(p + "self_attn.q_norm", cfg.head_dim, 1.0, 0.1)
                vector(p + "self_attn.k_norm", cfg.head_dim, 1.0, 0.1)
            if cfg.qkv_bias:
                vector(p + "self_attn.q_proj.bias", cfg.n_q, 0.0, 0.5)
                vector(p + "self_attn.k_proj.bias", cfg.n_kvd, 0.0, 0.5)
                vector(p + "self_attn.v_proj.bias", cfg.n_kvd, 0.0, 0.5)

    def set_embedding(self, embed_seed: int, embed_tau: float, loud_rows: int = 0, loud_gain: float = 1.0) -> None:
        c = self.cfg
        self.mats["embed_tokens"] = oracle.dense(
            oracle.synth_fill(c.vocab * c.hidden, embed_seed, 0.0, self.std, 4, row_len=c.hidden, tau=embed_tau,
                              loud_rows=loud_rows, loud_gain=loud_gain).reshape(c.vocab, c.hidden))


def loud_rows_equal(host_weights, rows: int, gain: float) -> np.ndarray:
    """Multiplies the first `rows` rows of a host model's (bf16, tied) embedding by `gain`, a power of two so that
    the product is exact: equally loud rows, where the generator's own loud rows halve from row to row.  Returns
    the changed rows (bf16 bits, [rows, hidden]) for the upload into the device model."""
    assert gain > 0 and float(np.log2(gain)).is_integer()
    emb = host_weights.mats["embed_tokens"]
    w = np.asarray(emb.w).reshape(emb.n, emb.k)
    w[:rows] = oracle.f32_to_bf16((oracle.bf16_to_f32(w[:rows]) * np.float32(gain)).astype(np.float32))
    return w[:rows].copy()


def host_weight(dw) -> oracle.QWeight:
    """Download a fusekit_amd DeviceWeight into an oracle QWeight (host weights pass through)."""
    if isinstance(dw, oracle.QWeight):
        return dw
    if dw.bits == 16:
        return oracle.dense(dw.w.to_numpy(np.uint16, (dw.n, dw.k)))
    per = 32 // dw.bits
    return oracle.QWeight(dw.w.to_numpy(np.uint32, (dw.n, dw.k // per)),
                          dw.scales.to_numpy(np.uint16, (dw.n, dw.k // dw.group)),
                          dw.biases.to_numpy(np.uint16, (dw.n, dw.k // dw.group)), dw.n, dw.k, dw.bits, dw.group)


class OracleDecoder:
    """CPU oracle of a dense decoder fed with the very bytes the GPU model holds."""

    def __init__(self, cfg, weights):
        import ctypes as C
        self.cfg = cfg
        self.keep = []
        u16p = C.POINTER(C.c_uint16)

        def vec(name):
            a = weights.vecs[name]
            a = a if isinstance(a, np.ndarray) else a.to_numpy(np.uint16)
            self.keep.append(a)
            return a.ctypes.data_as(u16p)

        def mat(name):
            W = host_weight(weights.mats[name])
            self.keep.append(W)
            return W.c

        null = C.cast(None, u16p)
        self.layers = (oracle.Layer * cfg.n_layers)()
        cache_elems = cfg.n_kv * cfg.capacity * cfg.head_dim
        for l in range(cfg.n_layers):
            p = f"layers.{l}."
            L = self.layers[l]
            L.input_norm, L.post_norm = vec(p + "input_layernorm"), vec(p + "post_attention_layernorm")
            L.wq, L.wk, L.wv = (mat(p + f"self_attn.{n}_proj") for n in "qkv")
            L.wo = mat(p + "self_attn.o_proj")
            L.wgate, L.wup, L.wdown = (mat(p + f"mlp.{n}_proj") for n in ("gate", "up", "down"))
            L.bq, L.bk, L.bv = ((vec(p + f"self_attn.{n}_proj.bias") for n in "qkv") if cfg.qkv_bias
                                else (null, null, null))
            L.q_norm, L.k_norm = ((vec(p + "self_attn.q_norm"), vec(p + "self_attn.k_norm")) if cfg.qk_norm
                                  else (null, null))
            if getattr(cfg, "kv_bits", 0):
                u32p = C.POINTER(C.c_uint32)
                K = oracle.QuantCache(cfg.n_kv, cfg.capacity, cfg.head_dim, cfg.kv_bits, cfg.kv_group)
                V = oracle.QuantCache(cfg.n_kv, cfg.capacity, cfg.head_dim, cfg.kv_bits, cfg.kv_group)
                self.keep += [K, V]
                L.ck_packed, L.ck_scales, L.ck_biases = (K.packed.ctypes.data_as(u32p), K.scales.ctypes.data_as(u16p),
                                                         K.biases.ctypes.data_as(u16p))
                L.cv_packed, L.cv_scales, L.cv_biases = (V.packed.ctypes.data_as(u32p), V.scales.ctypes.data_as(u16p),
                                                         V.biases.ctypes.data_as(u16p))
            else:
                ck, cv = np.zeros(cache_elems, np.uint16), np.zeros(cache_elems, np.uint16)
                self.keep += [ck, cv]
                L.cache_k, L.cache_v = ck.ctypes.data_as(u16p), cv.ctypes.data_as(u16p)
        emb = mat("embed_tokens")
        head = mat("lm_head") if "lm_head" in weights.mats else emb
        self.model = oracle.Model(cfg.n_layers, cfg.hidden, cfg.n_heads, cfg.n_kv, cfg.head_dim, cfg.inter, cfg.vocab,
                                  cfg.eps, cfg.theta, 1.0 / np.sqrt(cfg.head_dim), getattr(cfg, "embed_scale", 1.0), cfg.swiglu_variant,
                                  cfg.capacity, emb, head, vec("final_norm"), self.layers,
                                  getattr(cfg, "kv_bits", 0), getattr(cfg, "kv_group", 64))

    def step(self, token: int, offset: int, want_logits: bool = False):
        logits = np.empty(self.cfg.vocab, np.uint16) if want_logits else None
        nxt, margin = oracle.decoder_step(self.model, token, offset, logits)
        return nxt, margin, logits

    def generate(self, prompt, max_tokens):
        """Returns (tokens, margins): greedy tokens and the top-1/top-2 logit margin at each step."""
        toks, margins = [], []
        nxt = None
        for i, t in enumerate(prompt):
            nxt, m, _ = self.step(int(t), i)
        toks.append(nxt); margins.append(m)
        off = len(prompt)
        while len(toks) < max_tokens:
            nxt, m, _ = self.step(toks[-1], off)
            toks.append(nxt); margins.append(m)
            off += 1
        return toks, margins


class HostMoeWeights:
    """The mixture-of-experts decoder's weights built on the HOST with the oracle's copy of the library's
    host-reproducible generator and the oracle's quantiser: the bytes `MoeWeights.random_init(cfg, seed, std,
    exact=True, ...)` puts into HBM (same seed sequence).  `mats`: oracle QWeight / StackedWeight, `vecs`: bf16 bits."""

    def __init__(self, cfg, seed: int = 0, std: float = 0.02, embed_loud_rows: int = 0, embed_loud_gain: float = 1.0):
        self.cfg = c = cfg
        self.mats, self.vecs = {}, {}
        counter = [seed * 100003 + 7]

        def next_seed():
            counter[0] += 1
            return counter[0]

        def matrix(name, n, k, experts=0, sd=std):
            rows = n * max(experts, 1)
            W = oracle.quantize(oracle.synth_fill(rows * k, next_seed(), 0.0, sd, 3).reshape(rows, k), c.bits, c.group)
            if experts:
                S = oracle.StackedWeight.__new__(oracle.StackedWeight)
                oracle.QWeight.__init__(S, np.asarray(W.w).reshape(experts, n, -1), np.asarray(W.scales).reshape(experts, n, -1),
                                        np.asarray(W.biases).reshape(experts, n, -1), n, k, c.bits, c.group)
                S.n_experts = experts
                W = S
            self.mats[name] = W

        def dense_bf16(name, n, k, sd):
            if name == "embed_tokens":
                a = oracle.synth_fill(n * k, next_seed(), 0.0, sd, 4, row_len=k, loud_rows=embed_loud_rows, loud_gain=embed_loud_gain)
            else:
                a = oracle.synth_fill(n * k, next_seed(), 0.0, sd, 4)
            self.mats[name] = oracle.dense(a.reshape(n, k))

        def vector(name, n, mean, sd):
            self.vecs[name] = oracle.synth_fill(n, next_seed(), mean, sd, 4)

        dense_bf16("embed_tokens", c.vocab, c.hidden, std)
        vector("final_norm", c.hidden, 1.0, 0.1)
        for l in range(c.n_layers):
            p = f"layers.{l}."
            vector(p + "input_layernorm", c.hidden, 1.0, 0.1)
            vector(p + "post_attention_layernorm", c.hidden, 1.0, 0.1)
            matrix(p + "self_attn.q_proj", c.n_heads * c.qk_dim, c.hidden)
            matrix(p + "self_attn.kv_a_proj_with_mqa", c.kv_lora_rank + c.rope_dim, c.hidden)
            vector(p + "self_attn.kv_a_layernorm", c.kv_lora_rank, 1.0, 0.1)
            matrix(p + "self_attn.kv_b_proj", c.n_heads * (c.nope_dim + c.v_dim), c.kv_lora_rank)
            matrix(p + "self_attn.o_proj", c.hidden, c.n_heads * c.v_dim)
            if l < c.first_dense:
                matrix(p + "mlp.gate_proj", c.dense_inter, c.hidden)
                matrix(p + "mlp.up_proj", c.dense_inter, c.hidden)
                matrix(p + "mlp.down_proj", c.hidden, c.dense_inter)
            else:
                dense_bf16(p + "mlp.gate", c.n_experts, c.hidden, 0.05)
                for nm in ("gate_proj", "up_proj"):
                    matrix(p + f"mlp.switch_mlp.{nm}", c.moe_inter, c.hidden, c.n_experts)
                    matrix(p + f"mlp.shared_experts.{nm}", c.shared_inter, c.hidden)
                matrix(p + "mlp.switch_mlp.down_proj", c.hidden, c.moe_inter, c.n_experts)
                matrix(p + "mlp.shared_experts.down_proj", c.hidden, c.shared_inter)


def moe_class_channels(cfg, mats, vecs, n_classes: int, first_channel: int, level: float, ladder, route_noise: float,
                       perm_seed: int, loud_rows: int, loud_gain: float, loud_ratio: float):
    """Gives a mixture-of-experts model what a trained one has and a random one lacks -- persistent large
    activations and routers that read them -- in a form whose routes VARY: by token, by layer, and so by step.
    On the bf16 arrays of `mats` / `vecs` (oracle weights), in place:
      * token t belongs to class t % n_classes; the tied embedding's column first_channel + k holds `level` for the
        tokens of class k and 0 for the others (the class channel dominates every RMS norm input of the stack: its
        normalised value is about sqrt(hidden)); the final norm's weight of those channels becomes 0, so that the
        head never sees them;
      * each router keeps its random rows scaled by `route_noise`; in layer l the experts are cut into n_classes
        blocks of n_experts / n_classes by a permutation drawn from (perm_seed, l), and column first_channel + k
        holds ladder[i] / sqrt(hidden) for the i-th expert of block k (i < top_k) and 0 elsewhere: a token of class
        k routes to block k's first top_k experts in layer l, whatever else the stack has computed, with the
        ladder's gaps between the probabilities;
      * rows j < loud_rows of the embedding are scaled by loud_gain * loud_ratio^-j (a few dominant rows, as trained
        embeddings have; the class columns are written afterwards).
    Classes of the top_k experts never overlap inside a layer, so a group of tokens of c different classes touches
    c * top_k distinct experts there.  Returns (names of the arrays changed, expected routes [n_layers][n_classes]
    as sorted expert lists; entries of dense layers are None)."""
    assert cfg.n_experts % n_classes == 0 and cfg.n_experts // n_classes >= cfg.top_k and len(ladder) == cfg.top_k
    changed = ["embed_tokens", "final_norm"]
    E = np.asarray(mats["embed_tokens"].w).reshape(cfg.vocab, cfg.hidden)
    for j in range(loud_rows):
        g = np.float32(loud_gain * loud_ratio ** -j)
        E[j] = oracle.f32_to_bf16((oracle.bf16_to_f32(E[j]) * g).astype(np.float32))
    lvl = oracle.f32_to_bf16(np.array([level], np.float32))[0]
    cls = np.arange(cfg.vocab) % n_classes
    for k in range(n_classes):
        E[:, first_channel + k] = np.where(cls == k, lvl, np.uint16(0))
        vecs["final_norm"][first_channel + k] = 0
    u = float(np.sqrt(cfg.hidden))
    per = cfg.n_experts // n_classes
    expected = []
    for l in range(cfg.n_layers):
        if l < cfg.first_dense:
            expected.append(None)
            continue
        name = f"layers.{l}.mlp.gate"
        R = np.asarray(mats[name].w).reshape(cfg.n_experts, cfg.hidden)
        R[:] = oracle.f32_to_bf16((oracle.bf16_to_f32(R) * np.float32(route_noise)).astype(np.float32))
        perm = rng(perm_seed * 1000 + l).permutation(cfg.n_experts)
        rows = []
        for k in range(n_classes):
            col = np.zeros(cfg.n_experts, np.float32)
            chosen = perm[k * per: k * per + cfg.top_k]
            col[chosen] = np.asarray(ladder, np.float32) / np.float32(u)
            R[:, first_channel + k] = oracle.f32_to_bf16(col)
            rows.append(sorted(int(e) for e in chosen))
        expected.append(rows)
        changed.append(name)
    return changed, expected


class OracleMoeDecoder:
    """CPU oracle of the mixture-of-experts decoder with low-rank keys, composed from the oracle's
    per-kernel functions on the very bytes the GPU model holds, one call per dispatch of the GPU task list."""

    def __init__(self, cfg, weights):
        self.cfg = c = cfg
        host = isinstance(weights, HostMoeWeights)
        self.vec = dict(weights.vecs) if host else {k: v.to_numpy(np.uint16) for k, v in weights.vecs.items()}
        self.mat = {}
        for k, dw in weights.mats.items():
            if host:
                self.mat[k] = dw
                continue
            E = getattr(dw, "n_experts", 0)
            if not E:
                self.mat[k] = host_weight(dw)
                continue
            per = 32 // dw.bits
            wq = dw.w.to_numpy(np.uint32, (E, dw.n, dw.k // per))
            sc = dw.scales.to_numpy(np.uint16, (E, dw.n, dw.k // dw.group))
            bi = dw.biases.to_numpy(np.uint16, (E, dw.n, dw.k // dw.group))
            S = oracle.StackedWeight.__new__(oracle.StackedWeight)     # the arrays are stacked already: no copy
            oracle.QWeight.__init__(S, wq, sc, bi, dw.n, dw.k, dw.bits, dw.group)
            S.n_experts = E
            self.mat[k] = S
        self.ck = [np.zeros(c.n_heads * c.capacity * c.qk_dim, np.uint16) for _ in range(c.n_layers)]
        self.cv = [np.zeros(c.n_heads * c.capacity * c.v_dim, np.uint16) for _ in range(c.n_layers)]
        self.route_scale = oracle.f32_to_bf16(np.array([c.route_scale], np.float32))
        self.routes = []          # expert indices of the last step, per MoE layer
        self.forced = 0           # layers (over all steps) where the forced routes differed from the oracle's own
        self.router_drift = 0.0   # largest rel-L2 between the GPU's and the oracle's router logits of a layer

    def step(self, token: int, offset: int, want_logits: bool = False, forced_routes=None, gpu_router_logits=None):
        """forced_routes [n_layers, top_k] with gpu_router_logits [n_layers, n_experts]: follow the GPU's routes.
        Routing is a discrete function of the router logits, and those carry the stack's accumulated rounding
        drift, so near the k-th probability the GPU and the oracle may choose differently.  Checked instead:
        the GPU's logits are close to the oracle's, and its route is EXACTLY the oracle's router applied to the
        GPU's own logits; the oracle then continues with those experts and its own probabilities for them."""
        c, m, v = self.cfg, self.mat, self.vec
        x = oracle.embed_lookup(m["embed_tokens"], token)
        packed = c.nope_dim + c.v_dim
        self.routes = []
        for l in range(c.n_layers):
            p = f"layers.{l}."
            xn = oracle.rmsnorm(x, v[p + "input_layernorm"], c.eps)
            q = oracle.qgemv(m[p + "self_attn.q_proj"], xn)
            kva = oracle.qgemv(m[p + "self_attn.kv_a_proj_with_mqa"], xn)
            lat = oracle.rmsnorm(kva[:c.kv_lora_rank].copy(), v[p + "self_attn.kv_a_layernorm"], c.eps)
            kvb = oracle.qgemv(m[p + "self_attn.kv_b_proj"], lat)
            k_pe = kva[c.kv_lora_rank:].copy().reshape(1, c.rope_dim)
            oracle.kv_store_split(kvb, packed, k_pe, 1, kvb[c.nope_dim:], packed, c.n_heads, c.nope_dim, c.rope_dim, c.v_dim,
                                  c.rope_dim, c.rope_traditional, c.theta, offset, offset, c.capacity, self.ck[l], self.cv[l])
            # the GPU rotates the query's rope part in place (rounded to T) in the same launch
            qh = q.reshape(c.n_heads, c.qk_dim).copy()
            for h in range(c.n_heads):
                row_k, row_v = np.zeros(c.qk_dim, np.uint16), np.zeros(1, np.uint16)
                oracle.kv_store_split(qh[h, :c.nope_dim].copy(), c.nope_dim, qh[h, c.nope_dim:].copy(), 1, np.zeros(1, np.uint16), 1, 1,
                                      c.nope_dim, c.rope_dim, 1, c.rope_dim, c.rope_traditional, c.theta, offset, 0, 1, row_k, row_v)
                qh[h] = row_k
            att = oracle.sdpa_decode(qh.reshape(-1), self.ck[l], self.cv[l], c.n_heads, c.n_heads, c.qk_dim, c.v_dim, offset + 1,
                                     c.capacity, 1.0 / np.sqrt(c.qk_dim))
            x1 = oracle.linear_residual(m[p + "self_attn.o_proj"], att, x)
            post = v[p + "post_attention_layernorm"]
            if l < c.first_dense:
                mid = oracle.gateup_swiglu(x1, post, c.eps, m[p + "mlp.gate_proj"], m[p + "mlp.up_proj"], c.swiglu_variant)
                x = oracle.linear_residual(m[p + "mlp.down_proj"], mid, x1)
                continue
            xn = oracle.rmsnorm(x1, post, c.eps)
            logits = oracle.qgemv(m[p + "mlp.gate"], xn)
            idx, rw = oracle.softmax_topk_route(logits, c.top_k, self.route_scale)
            idx, rw = idx.reshape(-1), rw.reshape(-1)
            if forced_routes is not None:
                gl = np.ascontiguousarray(gpu_router_logits[l])
                fg, fo = oracle.bf16_to_f32(gl).astype(np.float64), oracle.bf16_to_f32(logits).astype(np.float64)
                self.router_drift = max(self.router_drift, float(np.linalg.norm(fg - fo) / np.linalg.norm(fo)))
                own_idx, _ = oracle.softmax_topk_route(gl, c.top_k, self.route_scale)
                assert set(own_idx.reshape(-1).tolist()) == set(forced_routes[l].tolist()), (l, own_idx, forced_routes[l])
                if set(forced_routes[l].tolist()) != set(idx.tolist()):
                    all_idx, all_w = oracle.softmax_topk_route(logits, c.n_experts - 1, self.route_scale)
                    prob = dict(zip(all_idx.reshape(-1).tolist(), oracle.bf16_to_f32(all_w.reshape(-1)).tolist()))
                    idx = forced_routes[l].astype(np.uint32)
                    rw = oracle.f32_to_bf16(np.array([prob.get(int(e), 0.0) for e in idx], np.float32))
                    self.forced += 1
            self.routes.append(idx.copy())
            h = oracle.routed_qmv_swiglu(xn.reshape(1, -1), m[p + "mlp.switch_mlp.gate_proj"], m[p + "mlp.switch_mlp.up_proj"],
                                         np.zeros(c.top_k, np.uint32), idx, None)
            smid = oracle.gateup_swiglu(xn, None, c.eps, m[p + "mlp.shared_experts.gate_proj"], m[p + "mlp.shared_experts.up_proj"],
                                        c.swiglu_variant)
            x = oracle.routed_qmv_reduce(h, m[p + "mlp.switch_mlp.down_proj"], idx, rw, x1.reshape(1, -1), 1, c.top_k,
                                         np.arange(c.top_k, dtype=np.uint32), smid, m[p + "mlp.shared_experts.down_proj"]).reshape(-1)
        logits = oracle.final_rmsnorm_lm_head(x, v["final_norm"], c.eps, m["embed_tokens"])
        return oracle.argmax(logits), oracle.top2_margin(logits), (logits if want_logits else None)

    def generate(self, prompt, max_tokens):
        toks, margins, nxt = [], [], None
        for i, t in enumerate(prompt):
            nxt, mg, _ = self.step(int(t), i)
        toks.append(nxt); margins.append(mg)
        off = len(prompt)
        while len(toks) < max_tokens:
            nxt, mg, _ = self.step(toks[-1], off)
            toks.append(nxt); margins.append(mg)
            off += 1
        return toks, margins
