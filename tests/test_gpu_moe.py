"""Routed-expert (mixture-of-experts) Q4_K path on the GPU against the CPU oracle, through the
C ABI: top_k_rows -> moe_gate -> moe_experts_gate_up_q4k -> moe_experts_down_q4k, the ids and
launch protocol of src/models/qwen3_5/moe.cpp:396-423, plus the *_rows forms that run a whole
chunk of tokens in one launch.  Routing (ids) must match exactly; routing weights, phi and the
routed sum are fp32-accumulate paths held to the 1e-3 bound of tests/util.py:rel_err."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import norm_err, rel_err, rms_err, run

pytestmark = pytest.mark.gpu
TOL = 1e-3
# The grouped (17 tokens and more) path: the expert weights enter the matrix cores exactly (as
# integers q * sc, the block's d and the min term applied in fp32), the activations as fp16 under
# a power-of-two row scale -- x, which these tests draw bf16-valued (exact in fp16), and phi, whose
# rounding is the error that remains.  Measured over the cases below: largest error 1.6e-4 to
# 4.8e-4 of the rms output, 1.7e-5 to 1.2e-4 in the 2-norm, the largest for a single token
# (fp32-valued x: up to 2.9e-3 / 3.0e-4).
GROUPED_RMS, GROUPED_NORM = 1.5e-3, 2e-4


def expert_tensors(g, experts, hidden, inter):
    gate = np.concatenate([synth.q4k_weights(g, inter, hidden) for _ in range(experts)])
    up = np.concatenate([synth.q4k_weights(g, inter, hidden) for _ in range(experts)])
    down = np.concatenate([synth.q4k_weights(g, hidden, inter) for _ in range(experts)])
    return gate, up, down


def silu(v):
    v = v.astype(np.float32)
    with np.errstate(over="ignore"):
        return (v / (np.float32(1) + np.exp(-v, dtype=np.float32))).astype(np.float32)


@pytest.mark.parametrize("experts,hidden,inter,top_k", [(16, 512, 256, 4), (8, 2048, 512, 8), (5, 256, 768, 2)])
def test_decode_row_matches_oracle(backend, experts, hidden, inter, top_k):
    g = synth.rng(experts * 100 + hidden + inter)
    gate, up, down = expert_tensors(g, experts, hidden, inter)
    x = synth.activations_bf16(g, 1, hidden)
    logits = g.standard_normal(size=(1, experts)).astype(np.float32)
    gs, ds = gate.size // experts, down.size // experts

    d_logits = backend.Upload(logits)
    d_ids, d_vals = backend.AllocateBuffer(4 * top_k), backend.AllocateBuffer(4 * top_k)
    run(backend, "top_k_rows", [d_logits, d_ids, d_vals], [1, experts, top_k, 0], grid=(1, 1, 1))
    d_x, d_wsh = backend.Upload(x), backend.Upload(synth.activations_f32(g, 1, hidden))
    d_wts, d_sig = backend.AllocateBuffer(4 * top_k), backend.AllocateBuffer(4)
    run(backend, "moe_gate", [d_vals, d_x, d_wsh, d_wts, d_sig], [top_k, hidden], grid=(1, 1, 1))
    d_gate, d_up, d_down = backend.Upload(gate), backend.Upload(up), backend.Upload(down)
    d_phi = backend.AllocateBuffer(4 * top_k * inter)
    run(backend, "moe_experts_gate_up_q4k", [d_x, d_gate, d_up, d_ids, d_phi], [hidden, inter, top_k, gs, gs],
        grid=((inter * top_k + 7) // 8, 1, 1))
    d_out = backend.Upload(np.full(hidden, 3.0, dtype=np.float32))
    run(backend, "moe_experts_down_q4k", [d_phi, d_down, d_ids, d_wts, d_out], [hidden, inter, top_k, ds, 0],
        grid=((hidden + 7) // 8, 1, 1))
    backend.Synchronize()

    ids = backend.CopyD2H(d_ids, dtype=np.uint32)
    vals = backend.CopyD2H(d_vals, dtype=np.float32)
    want_ids, want_vals = oracle.top_k_row(logits[0], top_k)
    assert np.array_equal(ids, want_ids) and np.array_equal(vals, want_vals)
    wts = backend.CopyD2H(d_wts, dtype=np.float32)
    want_wts = oracle.moe_gate(want_vals)
    assert np.allclose(wts, want_wts, rtol=1e-5) and abs(float(wts.sum()) - 1.0) < 1e-5
    sig = backend.CopyD2H(d_sig, dtype=np.float32)[0]
    wsh = backend.CopyD2H(d_wsh, dtype=np.float32)
    dot = float(np.dot(x[0].astype(np.float64), wsh.astype(np.float64)))
    assert abs(sig - 1.0 / (1.0 + np.exp(-dot))) < 1e-5

    phi = backend.CopyD2H(d_phi, dtype=np.float32).reshape(top_k, inter)
    for s, e in enumerate(want_ids):
        ge = oracle.gemm_q4k(x, gate[e * gs:(e + 1) * gs], 1, inter, hidden)[0]
        ue = oracle.gemm_q4k(x, up[e * gs:(e + 1) * gs], 1, inter, hidden)[0]
        assert rel_err(phi[s], silu(ge) * ue) <= TOL, (s, rel_err(phi[s], silu(ge) * ue))
    out = backend.CopyD2H(d_out, dtype=np.float32)
    ref = oracle.moe_batch_forward_q4k(x, want_ids, want_wts, gate, up, down, hidden, inter)[0]
    assert rel_err(out, ref) <= TOL, rel_err(out, ref)

    # accumulate = 1 adds the routed sum to what the output already holds
    run(backend, "moe_experts_down_q4k", [d_phi, d_down, d_ids, d_wts, d_out], [hidden, inter, top_k, ds, 1],
        grid=((hidden + 7) // 8, 1, 1))
    backend.Synchronize()
    twice = backend.CopyD2H(d_out, dtype=np.float32)
    assert rel_err(twice, 2 * ref) <= TOL


def forward_rows(backend, x, ids, wts, gate, up, down, hidden, inter, experts):
    rows, top_k = ids.shape
    gs, ds = gate.size // experts, down.size // experts
    d_x, d_ids, d_wts = backend.Upload(x), backend.Upload(ids), backend.Upload(wts)
    d_gate, d_up, d_down = backend.Upload(gate), backend.Upload(up), backend.Upload(down)
    d_phi = backend.AllocateBuffer(4 * rows * top_k * inter)
    d_out = backend.AllocateBuffer(4 * rows * hidden)
    run(backend, "moe_experts_gate_up_q4k_rows", [d_x, d_gate, d_up, d_ids, d_phi],
        [hidden, inter, top_k, gs, gs, rows], grid=((inter * top_k + 7) // 8, rows, 1))
    run(backend, "moe_experts_down_q4k_rows", [d_phi, d_down, d_ids, d_wts, d_out],
        [hidden, inter, top_k, ds, 0, rows], grid=((hidden + 7) // 8, rows, 1))
    backend.Synchronize()
    return backend.CopyD2H(d_out, dtype=np.float32).reshape(rows, hidden)


@pytest.mark.parametrize("rows,experts,hidden,inter,top_k", [(7, 16, 512, 256, 4), (16, 12, 256, 512, 3),
                                                             (8, 8, 2048, 512, 8)])   # the last: four weight rows a wavefront
def test_rows_match_oracle(backend, rows, experts, hidden, inter, top_k):
    g = synth.rng(rows + experts + hidden)
    gate, up, down = expert_tensors(g, experts, hidden, inter)
    x = synth.activations_bf16(g, rows, hidden)
    ids, vals = synth.moe_routing(g, rows, experts, top_k)
    wts = np.stack([oracle.moe_gate(v) for v in vals])
    ref = oracle.moe_batch_forward_q4k(x, ids, wts, gate, up, down, hidden, inter)
    got = forward_rows(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("rows,experts,hidden,inter,top_k", [(16, 16, 512, 256, 4), (17, 16, 512, 256, 4), (48, 16, 512, 256, 4),
                                                             (130, 6, 256, 512, 3), (300, 9, 512, 256, 2),
                                                             (33, 3, 256, 2048, 2)])
def test_rows_ids_around_the_grouping_threshold(backend, rows, experts, hidden, inter, top_k):
    """moe_experts_gate_up_q4k_rows + moe_experts_down_q4k_rows: 16 tokens run one exact pass per
    token, 17 and more are grouped by expert on the fp16 MFMA path (bounds as for
    moe_experts_ffn_q4k_rows); accumulate adds to what the output held."""
    g = synth.rng(rows * 5 + experts + hidden)
    gate, up, down = expert_tensors(g, experts, hidden, inter)
    x = synth.activations_bf16(g, rows, hidden)
    ids, vals = synth.moe_routing(g, rows, experts, top_k)
    ids[0, 0] = experts + 3              # out of range: clamped to the last expert in both regimes
    wts = np.stack([oracle.moe_gate(v) for v in vals])
    clamped = np.minimum(ids, experts - 1)
    ref = oracle.moe_batch_forward_q4k(x, clamped, wts, gate, up, down, hidden, inter)
    got = forward_rows(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    if rows < 17:
        assert rel_err(got, ref) <= TOL, rel_err(got, ref)
    else:
        assert rms_err(got, ref) <= GROUPED_RMS and norm_err(got, ref) <= GROUPED_NORM, (rms_err(got, ref), norm_err(got, ref))
    again = forward_rows(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert np.array_equal(again, got)


def test_config4_shapes(backend):
    """BASELINE configs[4]: 256 experts, hidden 2048, expert FFN 512, softmax top-8; M = 1
    (decode) and M = 512 (prefill chunk) in one launch each.  The M = 512 result is checked on
    sampled rows against the oracle, and every row must equal the same token run alone (the
    kernels treat rows independently)."""
    g = synth.rng(4)
    experts, hidden, inter, top_k = 256, 2048, 512, 8
    one = synth.q4k_weights(g, inter, hidden)          # distinct bytes per expert, cheaply
    gate = np.concatenate([np.roll(one, 977 * e) for e in range(experts)])
    up = np.concatenate([np.roll(one, 1931 * e + 5) for e in range(experts)])
    dn = synth.q4k_weights(g, hidden, inter)
    down = np.concatenate([np.roll(dn, 1409 * e + 3) for e in range(experts)])
    # rolled bytes are still valid Q4_K only in the quant area; regenerate headers per expert
    nb = gate.size // 144
    for t in (gate, up, down):
        blocks = t.reshape(-1, 144)
        hdr = synth.q4k_weights(g, 1, 256 * 64).reshape(-1, 144)[:, :16]
        blocks[:, :16] = np.tile(hdr, (blocks.shape[0] // hdr.shape[0] + 1, 1))[: blocks.shape[0]]
    assert nb == experts * inter * (hidden // 256)
    rows = 512
    x = synth.activations_bf16(g, rows, hidden)
    ids, vals = synth.moe_routing(g, rows, experts, top_k)
    wts = np.stack([oracle.moe_gate(v) for v in vals])
    # tokens picked greedily until every one of the 256 experts has been routed to (at least 64 of them)
    sample, seen = [0, 1, 100, 255, 256, 511], set()
    for r in sample:
        seen.update(int(e) for e in ids[r])
    order = [int(r) for r in g.permutation(rows)]
    while len(seen) < experts or len(sample) < 64:
        r = max(order[:64], key=lambda t: len(set(int(e) for e in ids[t]) - seen)) if len(seen) < experts else order[0]
        order.remove(r)
        if r not in sample:
            sample.append(r)
            seen.update(int(e) for e in ids[r])
    assert len(seen) == experts and len(sample) >= 64
    ref = oracle.moe_batch_forward_q4k(x[sample], ids[sample], wts[sample], gate, up, down, hidden, inter)
    # Up to 16 tokens the two row-batched ids take one exact fp32 pass per token.
    few = forward_rows(backend, x[:16], ids[:16], wts[:16], gate, up, down, hidden, inter, experts)
    assert rel_err(few[:2], ref[:2]) <= TOL, rel_err(few[:2], ref[:2])
    alone = forward_rows(backend, x[:1], ids[:1], wts[:1], gate, up, down, hidden, inter, experts)
    assert np.array_equal(alone[0], few[0])
    # The whole chunk: the same two ids now group the tokens by expert (fp16 MFMA), as the
    # one-call form does; both within the grouped path's bound of the oracle, and of each other
    # to rounding (they share every kernel but the one that applies silu).
    got = forward_rows(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert np.all(np.isfinite(got))
    assert rms_err(got[sample], ref) <= GROUPED_RMS, rms_err(got[sample], ref)
    assert rms_err(got[:16], few) <= GROUPED_RMS and norm_err(got[:16], few) <= GROUPED_NORM
    grouped = forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert rms_err(grouped[sample], ref) <= GROUPED_RMS, rms_err(grouped[sample], ref)
    assert rms_err(grouped, got) <= 1e-5, rms_err(grouped, got)


def forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts, accumulate=0, out0=None):
    rows, top_k = ids.shape
    gs, ds = gate.size // experts, down.size // experts
    d_x, d_ids, d_wts = backend.Upload(x), backend.Upload(ids), backend.Upload(wts)
    d_gate, d_up, d_down = backend.Upload(gate), backend.Upload(up), backend.Upload(down)
    d_out = backend.Upload(out0) if out0 is not None else backend.AllocateBuffer(4 * rows * hidden)
    run(backend, "moe_experts_ffn_q4k_rows", [d_x, d_gate, d_up, d_down, d_ids, d_wts, d_out],
        [hidden, inter, top_k, gs, gs, ds, rows, accumulate], grid=(1, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(d_out, dtype=np.float32).reshape(rows, hidden)


@pytest.mark.parametrize("rows,experts,hidden,inter,top_k", [(1, 8, 256, 256, 2), (40, 16, 512, 256, 4),
                                                             (130, 6, 256, 512, 3), (64, 3, 768, 256, 1), (90, 12, 256, 256, 2),
                                                             (48, 4, 256, 1024, 2), (40, 3, 256, 2048, 2),
                                                             (200, 4, 512, 512, 2)])
def test_grouped_ffn_matches_oracle(backend, rows, experts, hidden, inter, top_k):
    """moe_experts_ffn_q4k_rows: tokens grouped by expert, three grouped fp16-MFMA GEMMs with
    exact weights; x and phi are rounded to fp16 (bounds GROUPED_RMS, GROUPED_NORM above, with
    fp32-valued x checked at the end against the bound that rounding x to fp16 allows).  Experts that receive more
    than 32 tokens (they take 64 rows a pass, then what is left: about 65 and about 100 tokens an
    expert both occur) and experts that receive none both occur here.  An inner
    width of 1024 takes the narrower of the two row-resident kernels, 2048 the streamed grouped
    tiles (the rows of phi no longer fit LDS)."""
    g = synth.rng(rows * 3 + experts + hidden + inter)
    gate, up, down = expert_tensors(g, experts, hidden, inter)
    x = synth.activations_bf16(g, rows, hidden)
    ids, vals = synth.moe_routing(g, rows, experts, top_k)
    wts = np.stack([oracle.moe_gate(v) for v in vals])
    ref = oracle.moe_batch_forward_q4k(x, ids, wts, gate, up, down, hidden, inter)
    got = forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert rms_err(got, ref) <= GROUPED_RMS, rms_err(got, ref)
    assert norm_err(got, ref) <= GROUPED_NORM, norm_err(got, ref)
    base = g.standard_normal(size=(rows, hidden)).astype(np.float32)
    acc = forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts, accumulate=1, out0=base)
    assert np.array_equal(acc, base + got)
    # the sorted position of a pair may differ from run to run (atomics), its result may not
    again = forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert np.array_equal(again, got)
    # activations with all 24 bits: rounding x to fp16 (11 bits) is now the largest error
    xf = synth.activations_f32(g, rows, hidden)
    ref = oracle.moe_batch_forward_q4k(xf, ids, wts, gate, up, down, hidden, inter)
    got = forward_grouped(backend, xf, ids, wts, gate, up, down, hidden, inter, experts)
    assert rms_err(got, ref) <= 6e-3 and norm_err(got, ref) <= 6e-4, (rms_err(got, ref), norm_err(got, ref))


def test_grouped_ffn_small_block_scales(backend):
    """Block headers of the size real checkpoints have (1e-6 .. 1e-4, some below the fp16 normal
    range): the weights are not rounded at all (integer operands, d and dmin * mn applied in
    fp32 or as exact fp16 pairs), so the bound of the test above holds unchanged."""
    g = synth.rng(99)
    rows, experts, hidden, inter, top_k = 70, 6, 512, 256, 2
    tensors = []
    for t in expert_tensors(g, experts, hidden, inter):
        blk = t.reshape(-1, 144)
        for col in (0, 2):
            blk[:, col:col + 2] = g.uniform(1e-6, 1e-4, blk.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
        tensors.append(blk.reshape(-1))
    gate, up, down = tensors
    x = synth.activations_bf16(g, rows, hidden)
    ids, vals = synth.moe_routing(g, rows, experts, top_k)
    wts = np.stack([oracle.moe_gate(v) for v in vals])
    ref = oracle.moe_batch_forward_q4k(x, ids, wts, gate, up, down, hidden, inter)
    got = forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert rms_err(got, ref) <= GROUPED_RMS, rms_err(got, ref)
    assert norm_err(got, ref) <= GROUPED_NORM, norm_err(got, ref)


def test_grouped_ffn_skewed_routing(backend):
    """Every token to the same two experts (segments of 300 rows, ten row tiles each; all other
    experts empty), then duplicate and out-of-range ids in a token's list (clamped to the last
    expert, as the per-row ids do)."""
    g = synth.rng(4321)
    rows, experts, hidden, inter, top_k = 300, 9, 512, 256, 2
    gate, up, down = expert_tensors(g, experts, hidden, inter)
    x = synth.activations_bf16(g, rows, hidden)
    ids = np.tile(np.array([[6, 2]], np.uint32), (rows, 1))
    wts = g.uniform(0.1, 0.9, size=(rows, top_k)).astype(np.float32)
    ref = oracle.moe_batch_forward_q4k(x, ids, wts, gate, up, down, hidden, inter)
    got = forward_grouped(backend, x, ids, wts, gate, up, down, hidden, inter, experts)
    assert rms_err(got, ref) <= GROUPED_RMS and norm_err(got, ref) <= GROUPED_NORM
    odd = ids.copy()
    odd[0] = [4, 4]                      # the same expert twice
    odd[1] = [experts + 7, 0]            # out of range: clamped to experts - 1
    clamped = odd.copy()
    clamped[1, 0] = experts - 1
    ref = oracle.moe_batch_forward_q4k(x, clamped, wts, gate, up, down, hidden, inter)
    got = forward_grouped(backend, x, odd, wts, gate, up, down, hidden, inter, experts)
    assert rms_err(got, ref) <= GROUPED_RMS and norm_err(got, ref) <= GROUPED_NORM


@pytest.mark.parametrize("experts,hidden,inter,top_k,rows", [(16, 512, 256, 4, 1), (8, 2048, 512, 8, 1),
                                                              (5, 260, 768, 2, 3), (256, 2048, 512, 8, 2),
                                                              (24, 2048, 512, 8, 8)])   # the last: four weight rows a wavefront
def test_down_q6k_matches_oracle(backend, experts, hidden, inter, top_k, rows):
    """moe_experts_down_q6k (the reference loads it next to the Q4_K one,
    src/models/qwen3_5/moe.cpp:107-115): out[t] (+)= sum_slot wts[t][slot] * D_{ids[t][slot]} phi[t][slot],
    expert tensors Q6_K [hidden, inter]."""
    g = synth.rng(9000 + experts + hidden + inter + rows)
    down = np.concatenate([synth.q6k_weights(g, hidden, inter) for _ in range(experts)])
    ds = down.size // experts
    phi = synth.activations_f32(g, rows * top_k, inter).reshape(rows, top_k, inter)
    ids = np.stack([g.permutation(experts)[:top_k] for _ in range(rows)]).astype(np.uint32)
    wts = g.uniform(0.05, 1.0, size=(rows, top_k)).astype(np.float32)
    want = np.zeros((rows, hidden), np.float64)
    for t in range(rows):
        for s in range(top_k):
            e = int(ids[t, s])
            y = oracle.gemm_q6k(phi[t, s:s + 1], down[e * ds:(e + 1) * ds], 1, hidden, inter)[0]
            want[t] += np.float64(wts[t, s]) * y.astype(np.float64)
    d_phi, d_down = backend.Upload(phi), backend.Upload(down)
    d_ids, d_wts = backend.Upload(ids), backend.Upload(wts)
    prev = synth.activations_f32(g, rows, hidden)
    for accumulate in (0, 1):
        d_out = backend.Upload(prev.copy())
        if rows == 1:
            run(backend, "moe_experts_down_q6k", [d_phi, d_down, d_ids, d_wts, d_out],
                [hidden, inter, top_k, ds, accumulate], grid=((hidden + 7) // 8, 1, 1))
        else:
            run(backend, "moe_experts_down_q6k_rows", [d_phi, d_down, d_ids, d_wts, d_out],
                [hidden, inter, top_k, ds, accumulate, rows], grid=((hidden + 7) // 8, rows, 1))
        backend.Synchronize()
        got = backend.CopyD2H(d_out, dtype=np.float32).reshape(rows, hidden)
        ref = want + (prev.astype(np.float64) if accumulate else 0.0)
        base = want      # the bound is relative to the routed sum, not to what it is added to
        assert rel_err(got - (prev if accumulate else 0), base) <= TOL, (accumulate, rel_err(got, ref))


@pytest.mark.parametrize("n,idx", [(1, 0), (2048, 3), (5000, 7)])
def test_moe_scale_add_matches_reference_formula(backend, n, idx):
    """o = a + f[idx] * b (src/backends/rocm/rocm_kernels_basic.cpp:1932-1942): the shared expert's
    output scaled by its gate and added to the routed sum.  One multiply and one add per element;
    the device may contract them into a fused multiply-add, so the result is one of the two."""
    g = synth.rng(7000 + n)
    a = g.standard_normal(n).astype(np.float32)
    b = g.standard_normal(n).astype(np.float32)
    f = g.standard_normal(8).astype(np.float32)
    da, db, df = backend.Upload(a), backend.Upload(b), backend.Upload(f)
    do = backend.AllocateBuffer(4 * n)
    run(backend, "moe_scale_add", [da, db, df, do], [n, idx], grid=((n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(do, dtype=np.float32)
    separate = a + f[idx] * b                                                     # rounded product, then the sum
    fused = (a.astype(np.float64) + np.float64(f[idx]) * b.astype(np.float64)).astype(np.float32)
    assert np.all((got == separate) | (got == fused))
