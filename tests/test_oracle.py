"""Pins the CPU oracle (oracle/) without re-typing its formula.

Each check is chosen so that a plausible mistake fails it: a wrong mask offset or `<`
for `<=` fails the harmonic closed form and the SDPA lower-right comparison; a missing
max-subtraction fails the one-hot limit; a wrong normaliser fails row-stochasticity and
the uniform case; a transposed operand fails the brute force and the key-permutation
property; a wrong cls_len clamp fails the cls_len >= S equivalence.
"""
import math

import numpy as np
import pytest
import torch

from oracle import colsum_exact, colsum_ext_exact, naive_colsum, visible
from oracle.c_ref import colsum_ref, colsum_ref_ext

IMPLS = {
    "torch_naive": lambda q, k, **kw: naive_colsum(q, k, **kw).double().numpy(),
    "torch_exact": lambda q, k, **kw: colsum_exact(q, k, **kw).numpy(),
    "plain_c": lambda q, k, **kw: colsum_ref(q.numpy(), k.numpy(), **kw),
}


def _rand(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_against_golden_bruteforce(impl, golden):
    """Committed vectors from a pure-Python float64 brute force (tests/golden/make_golden.py)."""
    for name, c in golden.items():
        q = torch.from_numpy(c["q"].astype(np.float32))
        k = torch.from_numpy(c["k"].astype(np.float32))
        got = IMPLS[impl](q, k, scale=c["scale"], is_causal=c["causal"], cls_len=c["cls_len"])
        assert got.shape == c["out"].shape, name
        tol = 2e-6 if impl == "torch_naive" else 1e-6  # fp32 softmax vs float64
        np.testing.assert_allclose(got, c["out"], rtol=tol, atol=1e-9, err_msg=name)


@pytest.mark.parametrize("impl", sorted(IMPLS))
@pytest.mark.parametrize("sq,sk,causal", [(9, 9, False), (5, 12, True), (12, 5, True), (7, 7, True), (1, 9, True)])
def test_rows_are_stochastic(impl, sq, sk, causal):
    q, k = _rand((2 if not causal else 1, 3, sq, 8), 1), _rand((2 if not causal else 1, 3, sk, 8), 2)
    if not causal:
        k = k[:, :, :sq]
    out = IMPLS[impl](q, k, is_causal=causal)
    np.testing.assert_allclose(out.sum(-1), 1.0, rtol=0, atol=1e-6)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_uniform_when_queries_are_zero(impl):
    q, k = torch.zeros(2, 3, 11, 8), _rand((2, 3, 11, 8), 3)
    out = IMPLS[impl](q, k)
    np.testing.assert_allclose(out, 1.0 / 11, rtol=1e-6)


@pytest.mark.parametrize("impl", sorted(IMPLS))
@pytest.mark.parametrize("sq,sk", [(5, 12), (8, 8), (1, 6), (12, 5), (16, 40)])
def test_causal_alignment_closed_form(impl, sq, sk):
    """Q = 0 makes every row uniform over its visible keys, so the column means are
    harmonic sums fixed by the alignment alone: row i sees k_past + i + 1 keys (capped
    at S_k), with k_past = max(0, S_k - S_q)."""
    q, k = torch.zeros(1, 2, sq, 8), _rand((1, 2, sk, 8), 4)
    out = IMPLS[impl](q, k, is_causal=True)[0]
    k_past = max(0, sk - sq)
    want = np.zeros(sk)
    for i in range(sq):
        n = min(sk, k_past + i + 1)
        want[:n] += 1.0 / n
    want /= sq
    np.testing.assert_allclose(out, want, rtol=2e-6, atol=1e-12)


def test_mask_is_prefix_plus_lower_triangle():
    """The visibility predicate equals the construction the reference spells out
    (baselines.py:49-62): every prefix key visible, lower-triangular last window."""
    for sq, sk in [(5, 12), (5, 5), (1, 9), (16, 16), (3, 4)]:
        want = np.zeros((sq, sk), dtype=bool)
        past = sk - sq
        want[:, :past] = True
        want[:, past:] = np.tril(np.ones((sq, sq), dtype=bool))
        assert np.array_equal(visible(sq, sk).numpy(), want), (sq, sk)
    for sq, sk in [(9, 4), (12, 5)]:  # fewer keys than queries: plain k <= q
        want = np.arange(sk)[None, :] <= np.arange(sq)[:, None]
        assert np.array_equal(visible(sq, sk).numpy(), want), (sq, sk)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_matches_library_attention_with_identity_values(impl):
    """scaled_dot_product_attention with V = I returns the attention matrix itself:
    an independent library implementation of softmax(QK^T * scale) and of the
    lower-right aligned causal mask."""
    import torch.nn.functional as F
    from torch.nn.attention.bias import causal_lower_right

    q, k = _rand((2, 3, 10, 16), 5).double(), _rand((2, 3, 10, 16), 6).double()
    attn = F.scaled_dot_product_attention(q, k, torch.eye(10, dtype=torch.float64).expand(2, 3, 10, 10), scale=0.3)
    np.testing.assert_allclose(IMPLS[impl](q.float(), k.float(), scale=0.3), attn.mean((1, 2)).numpy(), rtol=3e-6)
    # cls_len = c is the same matrix restricted to its first c rows
    np.testing.assert_allclose(IMPLS[impl](q.float(), k.float(), scale=0.3, cls_len=4),
                               attn[:, :, :4].mean((1, 2)).numpy(), rtol=3e-6)
    qc, kc = _rand((1, 2, 6, 16), 7).double(), _rand((1, 2, 17, 16), 8).double()
    attn = F.scaled_dot_product_attention(qc, kc, torch.eye(17, dtype=torch.float64).expand(1, 2, 17, 17),
                                          attn_mask=causal_lower_right(6, 17), scale=0.2)
    np.testing.assert_allclose(IMPLS[impl](qc.float(), kc.float(), scale=0.2, is_causal=True),
                               attn.mean((1, 2)).numpy(), rtol=3e-6, atol=1e-12)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_cls_len_clamps_and_reduces_to_a_gemv(impl):
    q, k = _rand((2, 3, 9, 8), 9), _rand((2, 3, 9, 8), 10)
    full = IMPLS[impl](q, k)
    np.testing.assert_allclose(IMPLS[impl](q, k, cls_len=9), full, rtol=1e-6)
    np.testing.assert_allclose(IMPLS[impl](q, k, cls_len=500), full, rtol=1e-6)
    # cls_len = 1: softmax(K q0 * scale) averaged over heads
    s = torch.einsum("bhd,bhkd->bhk", q[:, :, 0].double(), k.double()) / math.sqrt(8)
    want = torch.softmax(s, -1).mean(1).numpy()
    np.testing.assert_allclose(IMPLS[impl](q, k, cls_len=1), want, rtol=3e-6)
    with pytest.raises(ValueError):
        naive_colsum(q, k, cls_len=0)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_invariances(impl):
    q, k = _rand((2, 3, 12, 8), 11), _rand((2, 3, 12, 8), 12)
    base = IMPLS[impl](q, k, scale=0.4)
    # adding the same vector to every key shifts each row's scores by a constant
    shifted = IMPLS[impl](q, k + _rand((2, 3, 1, 8), 13), scale=0.4)
    np.testing.assert_allclose(shifted, base, rtol=2e-5)
    # (cQ, scale/c) == (Q, scale)
    np.testing.assert_allclose(IMPLS[impl](q * 4.0, k, scale=0.1), base, rtol=2e-6)
    # permuting keys permutes the output; permuting heads or query rows does nothing
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(0))
    np.testing.assert_allclose(IMPLS[impl](q, k[:, :, perm], scale=0.4), base[:, perm.numpy()], rtol=2e-6)
    np.testing.assert_allclose(IMPLS[impl](q[:, [2, 0, 1]], k[:, [2, 0, 1]], scale=0.4), base, rtol=2e-6)
    np.testing.assert_allclose(IMPLS[impl](q[:, :, perm], k, scale=0.4), base, rtol=2e-6)
    # default scale is 1/sqrt(D)
    np.testing.assert_allclose(IMPLS[impl](q, k), IMPLS[impl](q, k, scale=8 ** -0.5), rtol=1e-7)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_one_hot_limit_at_huge_scale(impl):
    """scale -> large: each row puts all its mass on its arg-max key; needs the
    max-subtraction to avoid overflow."""
    q, k = _rand((1, 2, 10, 8), 14), _rand((1, 2, 10, 8), 15)
    out = IMPLS[impl](q, k, scale=1.0e5)[0]
    winners = (q.double() @ k.double().transpose(-1, -2)).argmax(-1).reshape(-1).numpy()
    want = np.bincount(winners, minlength=10) / 20.0
    np.testing.assert_allclose(out, want, atol=1e-9)


def test_single_causal_query_sees_every_key():
    """Q_len = 1 is aligned to the last key, so the causal result is the plain softmax row."""
    q, k = _rand((1, 2, 1, 8), 16), _rand((1, 2, 13, 8), 17)
    s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(8)
    want = torch.softmax(s, -1).mean((1, 2)).numpy()
    for impl in IMPLS.values():
        np.testing.assert_allclose(impl(q, k, is_causal=True), want, rtol=3e-6)


def test_fp32_reference_leaves_the_bar_at_huge_scores():
    """Where |scale * score| reaches the tens of thousands one fp32 ulp of a score is worth 1e-3 of a
    probability: the fp32 eager path (the parity target) is then itself an order of magnitude
    further from float64 than at ordinary magnitudes, within |scale| * ulp_fp32(max |score|).
    This is the edge of the domain in which the 1e-3 relative bar can be asked of an fp32 evaluation."""
    q, k = (_rand((1, 2, 256, 128), 31) * 4).half().float(), (_rand((1, 2, 256, 128), 32) * 4).half().float()
    exact = colsum_exact(q, k, scale=20.0).numpy()
    eager = naive_colsum(q, k, scale=20.0).double().numpy()
    rel = np.max(np.abs(eager - exact) / np.maximum(np.abs(exact), 1e-12))
    s_max = float((q.double() @ k.double().transpose(-1, -2)).abs().max())
    ulp = 2.0 ** (math.floor(math.log2(s_max)) - 23)
    assert 1e-5 < rel <= 20.0 * ulp * 1.5, (rel, s_max)
    # at ordinary magnitudes the same comparison is at fp32 rounding level
    q, k = q / 4, k / 4
    rel = np.max(np.abs(naive_colsum(q, k).double().numpy() - colsum_exact(q, k).numpy()) / colsum_exact(q, k).numpy())
    assert rel < 2e-6


# ---------------------------------------------------------------------------------------
# beyond the reference operator's domain: grouped key heads, batched causal, causal cls_len,
# explicit k_past, S_q != S_k
# ---------------------------------------------------------------------------------------
EXT_IMPLS = {
    "torch_ext": lambda q, k, **kw: colsum_ext_exact(q, k, **kw).numpy(),
    "plain_c_ext": lambda q, k, **kw: colsum_ref_ext(q.numpy(), k.numpy(), **kw),
}


@pytest.mark.parametrize("impl", sorted(EXT_IMPLS))
def test_ext_against_golden_bruteforce(impl, golden_ext):
    for name, c in golden_ext.items():
        q = torch.from_numpy(c["q"].astype(np.float32))
        k = torch.from_numpy(c["k"].astype(np.float32))
        got = EXT_IMPLS[impl](q, k, scale=c["scale"], is_causal=c["causal"], cls_len=c["cls_len"], k_past=c["k_past"])
        np.testing.assert_allclose(got, c["out"], rtol=1e-6, atol=1e-9, err_msg=name)


@pytest.mark.parametrize("impl", sorted(EXT_IMPLS))
def test_ext_reduces_to_the_pinned_oracle(impl, golden):
    """Without grouping, batching of causal calls or a causal cls_len it is the reference's definition."""
    for name, c in golden.items():
        q = torch.from_numpy(c["q"].astype(np.float32))
        k = torch.from_numpy(c["k"].astype(np.float32))
        got = EXT_IMPLS[impl](q, k, scale=c["scale"], is_causal=c["causal"], cls_len=c["cls_len"])
        np.testing.assert_allclose(got, c["out"], rtol=1e-6, atol=1e-9, err_msg=name)


@pytest.mark.parametrize("impl", sorted(EXT_IMPLS))
def test_ext_matches_library_grouped_attention(impl):
    """scaled_dot_product_attention(enable_gqa=True) with V = I: the library's own grouping of
    query heads over key heads, with and without its lower-right causal bias, batch of 2."""
    import torch.nn.functional as F
    from torch.nn.attention.bias import causal_lower_right

    q, k = _rand((2, 6, 9, 16), 21).double(), _rand((2, 2, 14, 16), 22).double()
    eye = torch.eye(14, dtype=torch.float64).expand(2, 2, 14, 14)
    attn = F.scaled_dot_product_attention(q, k, eye, scale=0.3, enable_gqa=True)
    np.testing.assert_allclose(EXT_IMPLS[impl](q.float(), k.float(), scale=0.3), attn.mean((1, 2)).numpy(), rtol=3e-6)
    attn = F.scaled_dot_product_attention(q, k, eye, attn_mask=causal_lower_right(9, 14), scale=0.3, enable_gqa=True)
    np.testing.assert_allclose(EXT_IMPLS[impl](q.float(), k.float(), scale=0.3, is_causal=True),
                               attn.mean((1, 2)).numpy(), rtol=3e-6, atol=1e-12)
    # causal cls_len = c: the same matrix restricted to its first c rows
    np.testing.assert_allclose(EXT_IMPLS[impl](q.float(), k.float(), scale=0.3, is_causal=True, cls_len=4),
                               attn[:, :, :4].mean((1, 2)).numpy(), rtol=3e-6, atol=1e-12)
    # the grouping is repeat_interleave of the key heads
    want = np.stack([colsum_exact(q[b:b + 1].float(), k[b:b + 1].float().repeat_interleave(3, dim=1), scale=0.3,
                                  is_causal=True).numpy()[0] for b in range(2)])
    np.testing.assert_allclose(EXT_IMPLS[impl](q.float(), k.float(), scale=0.3, is_causal=True), want, rtol=1e-6)


@pytest.mark.parametrize("impl", sorted(EXT_IMPLS))
@pytest.mark.parametrize("sq,sk,k_past,cls_len", [(5, 12, 3, None), (6, 20, 0, 4), (4, 9, 30, None), (8, 8, 2, 3)])
def test_ext_causal_closed_form_with_explicit_k_past(impl, sq, sk, k_past, cls_len):
    """Q = 0: row i is uniform over its min(S_k, k_past + i + 1) visible keys; harmonic sums fix
    k_past, the <= and the normaliser over the averaged rows."""
    q, k = torch.zeros(2, 4, sq, 8), _rand((2, 2, sk, 8), 23)
    out = EXT_IMPLS[impl](q, k, is_causal=True, k_past=k_past, cls_len=cls_len)
    rows = sq if cls_len is None else min(cls_len, sq)
    want = np.zeros(sk)
    for i in range(rows):
        n = min(sk, k_past + i + 1)
        want[:n] += 1.0 / n
    want /= rows
    np.testing.assert_allclose(out, np.stack([want, want]), rtol=2e-6, atol=1e-12)
