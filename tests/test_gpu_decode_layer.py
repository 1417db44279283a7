"""GPU: the Q8_0 launches of one decode layer chained through the C ABI, against the CPU checker's chain.

token embedding (get_rows) -> [RMS norm * weight -> quantize -> q/k/v mat-vecs] (one launch) -> o mat-vec -> residual ->
[RMS norm * weight -> quantize -> gate/up -> SiLU * up -> quantize -> down -> + residual] (one launch), the order of the
reference's graph (infra/core_traits.hpp:570-594, :768-769, :953-1052) with the attention itself left out (its output is
stood in for by the query vector: attention is not part of this path).  Every stage is checked against the checker fed
with the GPU's own previous stage (tight bound), and the end of the chain against the checker's own chain (the bound
that allows for quantizers between stages amplifying last-bit differences).
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

END_TO_END_TOL = 2e-3  # three quantizers between the embedding and the layer output


def _cpu_norm_quant(oracle, x, w, eps):
    return oracle.rms_norm_quantize_rows(x[None, :], w, eps)[0]


@pytest.mark.parametrize("hidden,n_kv,n_ff,vocab", [(512, 128, 1536, 1000), (4096, 1024, 14336, 4000)])
def test_decode_layer_chain(q8, oracle, hidden, n_kv, n_ff, vocab):
    rng = np.random.default_rng(hidden + n_ff)
    eps = 1e-5
    # block scales chosen so that every projection has about unit gain (quants are uniform in [-127, 127], rms 73): values stay
    # O(1) through the chain instead of growing by sqrt(K) * 73 * sigma per stage
    def sigma(k_in):
        return 1.0 / (58.0 * np.sqrt(k_in))

    emb = random_blocks(rng, vocab, hidden, 1.0 / 58.0)
    wq, wk, wv, wo = (random_blocks(rng, n, hidden, sigma(hidden)) for n in (hidden, n_kv, n_kv, hidden))
    wg, wu, wd = random_blocks(rng, n_ff, hidden, sigma(hidden)), random_blocks(rng, n_ff, hidden, sigma(hidden)), random_blocks(rng, hidden, n_ff, sigma(n_ff))
    attn_norm = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    ffn_norm = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    token = int(rng.integers(0, vocab))

    t = {name: q8.tile(to_dev(w), n, k) for name, (w, n, k) in {
        "emb": (emb, vocab, hidden), "q": (wq, hidden, hidden), "k": (wk, n_kv, hidden), "v": (wv, n_kv, hidden), "o": (wo, hidden, hidden),
        "g": (wg, n_ff, hidden), "u": (wu, n_ff, hidden), "d": (wd, hidden, n_ff)}.items()}

    # ---- GPU chain ----
    import torch

    ids = torch.tensor([token], dtype=torch.int32, device="cuda")
    x0 = q8.get_rows(t["emb"], ids, vocab, hidden, tiled=True).reshape(-1)
    q, k_, v = q8.gemv_f32([t["q"], t["k"], t["v"]], x0, [hidden, n_kv, n_kv], hidden, norm_weight=to_dev(attn_norm), eps=eps)
    h = q8.gemv_residual_f32(t["o"], q, x0, hidden, hidden)  # the attention output is stood in for by q; residual add inside the launch
    o = h - x0
    y = q8.ffn(t["g"], t["u"], t["d"], h, n_ff, hidden, hidden, residual=h, norm_weight=to_dev(ffn_norm), eps=eps)

    # ---- stage by stage: the checker on the GPU's own inputs ----
    x0_cpu = oracle.get_rows(emb, np.array([token], np.int32), vocab, hidden)[0][0]
    assert np.array_equal(to_host(x0), x0_cpu)  # one fp32 multiply per element: bit-exact
    xq = _cpu_norm_quant(oracle, to_host(x0), attn_norm, eps)
    for got, w, n in ((q, wq, hidden), (k_, wk, n_kv), (v, wv, n_kv)):
        assert rel_l2(to_host(got), oracle.gemv(w, xq, n, hidden)) <= REL_L2_TOL
    assert rel_l2(to_host(h), oracle.gemv(wo, oracle.quantize_rows(to_host(q))[0], hidden, hidden) + x0_cpu) <= REL_L2_TOL
    del o
    hq = _cpu_norm_quant(oracle, to_host(h), ffn_norm, eps)
    g_gpu, u_gpu = (to_host(a) for a in q8.debug_ffn_gate_up(n_ff))
    assert rel_l2(g_gpu, oracle.gemv(wg, hq, n_ff, hidden)) <= REL_L2_TOL and rel_l2(u_gpu, oracle.gemv(wu, hq, n_ff, hidden)) <= REL_L2_TOL
    aq = oracle.silu_mul_quantize_rows(g_gpu, u_gpu)[0]
    assert rel_l2(to_host(y), oracle.gemv(wd, aq, hidden, n_ff) + to_host(h)) <= REL_L2_TOL

    # ---- the checker's own chain, end to end ----
    q_c = oracle.gemv(wq, _cpu_norm_quant(oracle, x0_cpu, attn_norm, eps), hidden, hidden)
    o_c = oracle.gemv(wo, oracle.quantize_rows(q_c)[0], hidden, hidden)
    h_c = x0_cpu + o_c
    hq_c = _cpu_norm_quant(oracle, h_c, ffn_norm, eps)
    a_c = oracle.silu_mul_quantize_rows(oracle.gemv(wg, hq_c, n_ff, hidden), oracle.gemv(wu, hq_c, n_ff, hidden))[0]
    y_c = oracle.gemv(wd, a_c, hidden, n_ff) + h_c
    assert rel_l2(to_host(y), y_c) <= END_TO_END_TOL
    assert np.isfinite(to_host(y)).all()


@pytest.mark.parametrize("m,hidden,n_kv,n_ff,vocab", [(40, 512, 128, 1536, 1000), (130, 1024, 256, 2816, 3000)])
def test_prefill_layer_chain(q8, oracle, m, hidden, n_kv, n_ff, vocab):
    # the same layer for M prompt tokens: get_rows -> RMS norm * weight -> quantize (one kernel, tiled output shared by q/k/v)
    # -> mat-mats -> o -> residual -> RMS norm * weight -> quantize -> gate/up mat-mats -> SiLU * up -> quantize -> down
    rng = np.random.default_rng(m + hidden)
    eps = 1e-5

    def sigma(k_in):
        return 1.0 / (58.0 * np.sqrt(k_in))

    emb = random_blocks(rng, vocab, hidden, 1.0 / 58.0)
    wq, wk, wo = (random_blocks(rng, n, hidden, sigma(hidden)) for n in (hidden, n_kv, hidden))
    wg, wu, wd = random_blocks(rng, n_ff, hidden, sigma(hidden)), random_blocks(rng, n_ff, hidden, sigma(hidden)), random_blocks(rng, hidden, n_ff, sigma(n_ff))
    attn_norm = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    ffn_norm = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    tokens = rng.integers(0, vocab, size=m).astype(np.int32)
    t = {name: q8.tile(to_dev(w), n, k) for name, (w, n, k) in {
        "emb": (emb, vocab, hidden), "q": (wq, hidden, hidden), "k": (wk, n_kv, hidden), "o": (wo, hidden, hidden),
        "g": (wg, n_ff, hidden), "u": (wu, n_ff, hidden), "d": (wd, hidden, n_ff)}.items()}

    def cpu_mm(w, aq, n, k):
        return oracle.gemm(w, aq, m, n, k, threads=4) if (k // 32) % 16 == 0 else oracle.gemm(w, aq, m, n, k)

    # ---- GPU chain ----
    x0 = q8.get_rows(t["emb"], to_dev(tokens), vocab, hidden, tiled=True)
    a0 = q8.rms_norm_quantize(x0, to_dev(attn_norm), eps, tiled=True)
    q = q8.gemm(t["q"], a0, m, hidden, hidden, tiled=True)
    k_ = q8.gemm(t["k"], a0, m, n_kv, hidden, tiled=True)
    o = q8.mul_mat(t["o"], q, hidden, hidden)  # attention stood in for by q; quantize + mat-mat in one call
    h = x0 + o
    a1 = q8.rms_norm_quantize(h, to_dev(ffn_norm), eps, tiled=True)
    g = q8.gemm(t["g"], a1, m, n_ff, hidden, tiled=True)
    u = q8.gemm(t["u"], a1, m, n_ff, hidden, tiled=True)
    a2 = q8.silu_mul_quantize(g, u, tiled=True)
    y = q8.gemm_residual(t["d"], a2, h, m, hidden, n_ff)  # the down projection with the layer's second residual add in its store

    # ---- stage by stage on the GPU's own inputs: quantized activations bit for bit, fp32 outputs within the contract ----
    x0_cpu = oracle.get_rows(emb, tokens, vocab, hidden)[0]
    assert np.array_equal(to_host(x0), x0_cpu)
    a0_cpu = oracle.rms_norm_quantize_rows(to_host(x0), attn_norm, eps)
    assert np.array_equal(to_host(q8.untile(a0, m, hidden)).reshape(m, -1), a0_cpu)
    assert rel_l2(to_host(q), cpu_mm(wq, a0_cpu, hidden, hidden)) <= REL_L2_TOL
    assert rel_l2(to_host(k_), cpu_mm(wk, a0_cpu, n_kv, hidden)) <= REL_L2_TOL
    assert rel_l2(to_host(o), cpu_mm(wo, oracle.quantize_rows(to_host(q)), hidden, hidden)) <= REL_L2_TOL
    a1_cpu = oracle.rms_norm_quantize_rows(to_host(h), ffn_norm, eps)
    assert np.array_equal(to_host(q8.untile(a1, m, hidden)).reshape(m, -1), a1_cpu)
    assert rel_l2(to_host(g), cpu_mm(wg, a1_cpu, n_ff, hidden)) <= REL_L2_TOL
    a2_cpu = oracle.silu_mul_quantize_rows(to_host(g), to_host(u))
    assert np.array_equal(to_host(q8.untile(a2, m, n_ff)).reshape(m, -1), a2_cpu)
    assert rel_l2(to_host(y), cpu_mm(wd, a2_cpu, hidden, n_ff) + to_host(h)) <= REL_L2_TOL

    # ---- the checker's own chain ----
    q_c = cpu_mm(wq, oracle.rms_norm_quantize_rows(x0_cpu, attn_norm, eps), hidden, hidden)
    h_c = x0_cpu + cpu_mm(wo, oracle.quantize_rows(q_c), hidden, hidden)
    a1_c = oracle.rms_norm_quantize_rows(h_c, ffn_norm, eps)
    a2_c = oracle.silu_mul_quantize_rows(cpu_mm(wg, a1_c, n_ff, hidden), cpu_mm(wu, a1_c, n_ff, hidden))
    y_c = cpu_mm(wd, a2_c, hidden, n_ff) + h_c
    assert rel_l2(to_host(y), y_c) <= END_TO_END_TOL
