"""Pins the CPU oracle: closed forms, library routines, brute force, the C restatement
and the golden vectors held by the reference's own tests.  No GPU involved."""
import itertools
import math

import numpy as np
import pytest
import torch

from oracle import acache_oracle as O
from oracle import c_oracle as C


def _bits(t):
    return t.view(torch.int16) if t.dtype == torch.bfloat16 else t.view(torch.int32)


# ----------------------------------------------------------------------- RoPE
@pytest.mark.parametrize("theta,D", [(1e4, 64), (5e5, 128), (1e6, 128)])
def test_rope_table_against_float64(theta, D):
    cos, sin = O.rope_table(300, D, theta)
    # exact float64 angles; fp32 rounding of inv_freq and of the product moves the
    # angle by <= 2 ulp relative, i.e. <= (p+1)*2.5e-7 absolute in cos/sin
    j = np.arange(0, D, 2, dtype=np.float64)
    ang = np.arange(300, dtype=np.float64)[:, None] * (float(theta) ** (-j / D))[None, :]
    tol = (np.arange(300, dtype=np.float64)[:, None] + 1) * 2.5e-7
    assert cos.shape == (300, D) and sin.shape == (300, D)
    assert np.all(np.abs(cos[:, : D // 2].numpy() - np.cos(ang)) <= tol)
    assert np.all(np.abs(sin[:, : D // 2].numpy() - np.sin(ang)) <= tol)
    # cat(freqs, freqs): both halves identical
    assert torch.equal(cos[:, : D // 2], cos[:, D // 2:])
    assert torch.equal(sin[:, : D // 2], sin[:, D // 2:])
    # row 0 is the identity rotation
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)


def test_rope_table_matches_c_restatement():
    cos, sin = O.rope_table(1300, 128, 5e5)
    c_cos, c_sin = C.rope_table(1300, 128, 5e5)
    # libm vs torch vector math may differ in the last bits of the fp32 angle's cos/sin
    np.testing.assert_allclose(cos.numpy(), c_cos, atol=3e-4, rtol=0)
    np.testing.assert_allclose(sin.numpy(), c_sin, atol=3e-4, rtol=0)
    assert np.abs(cos.numpy()[:50] - c_cos[:50]).max() < 1e-6


def test_rot_half_is_a_quarter_turn():
    x = torch.randn(3, 2, 8)
    assert torch.equal(O.rot_half(O.rot_half(x)), -x)
    assert torch.equal(O.rot_half(x)[..., :4], -x[..., 4:])
    assert torch.equal(O.rot_half(x)[..., 4:], x[..., :4])


def test_rotation_closed_forms_fp32():
    torch.manual_seed(0)
    D = 128
    cos, sin = O.rope_table(2048, D, 5e5)
    x = torch.randn(40, 4, D)
    zero = torch.zeros(40, dtype=torch.long)
    # R(0) = I, bit exact
    assert torch.equal(O.rotate(x, zero, cos, sin), x)
    a = torch.randint(1, 900, (40,))
    b = torch.randint(1, 900, (40,))
    # R(a)R(b) = R(a+b)
    lhs = O.rotate(O.rotate(x, a, cos, sin), b, cos, sin)
    rhs = O.rotate(x, a + b, cos, sin)
    torch.testing.assert_close(lhs, rhs, atol=2e-4, rtol=0)
    # R(-d)R(d) = I
    back = O.rotate(O.rotate(x, a, cos, sin), -a, cos, sin)
    torch.testing.assert_close(back, x, atol=5e-6, rtol=0)
    # pair norms x_d^2 + x_{d+D/2}^2 are preserved
    y = O.rotate(x, a, cos, sin)
    n0 = x[..., : D // 2] ** 2 + x[..., D // 2:] ** 2
    n1 = y[..., : D // 2] ** 2 + y[..., D // 2:] ** 2
    torch.testing.assert_close(n0, n1, atol=1e-5, rtol=1e-5)
    # a wrong sign of rot_half or of sin would break this: explicit 2x2 rotation in float64
    ang = (a.double()[:, None] * (1.0 / (5e5 ** (torch.arange(0, D, 2).double() / D)))[None, :])
    x1, x2 = x[..., : D // 2].double(), x[..., D // 2:].double()
    e1 = x1 * ang.cos()[:, None] - x2 * ang.sin()[:, None]
    e2 = x2 * ang.cos()[:, None] + x1 * ang.sin()[:, None]
    torch.testing.assert_close(y.double(), torch.cat((e1, e2), -1), atol=2e-3, rtol=0)


def test_query_side_identity_ties_it_to_key_side():
    torch.manual_seed(1)
    D = 64
    cos, sin = O.rope_table(64, D)
    q = torch.randn(5, 2, D)
    k = torch.randn(5, 2, D)
    s = 11
    lhs = (O.rotate_query_inverse(q, s, cos, sin) * k).sum(-1)
    rhs = (q * O.rotate(k, torch.full((5,), s), cos, sin)).sum(-1)
    torch.testing.assert_close(lhs, rhs, atol=1e-4, rtol=1e-5)


def test_relocated_key_equals_raw_key_rotated_to_final_position_within_one_bf16_ulp():
    """Geometry of the reference's test_acache_relocates_shared_post_rope_keys
    (tests/test_attention_kernels.py:294-368): cache at position p, shift by d."""
    torch.manual_seed(2)
    D = 128
    cos, sin = O.rope_table(2600, D, 5e5)
    raw = torch.randn(64, 2, D)
    p = torch.randint(0, 1200, (64,))
    d = torch.randint(1, 1200, (64,))
    cached = O.rotate(raw, p, cos, sin).to(torch.bfloat16)
    moved = O.rotate(cached, d, cos, sin)
    direct = O.rotate(raw, p + d, cos, sin)
    err = (moved.float() - direct).abs()
    ulp = torch.maximum(direct.abs(), torch.tensor(2.0 ** -126)).log2().floor().exp2() * 2.0 ** -7
    # one bf16 rounding of the cached key (amplified by <= sqrt(2)) plus one of the result
    assert torch.all(err <= 2.5 * torch.maximum(ulp, ulp.amax(-1, keepdim=True)))


def test_negative_shift_is_inverse_sign_rule():
    torch.manual_seed(3)
    cos, sin = O.rope_table(32, 64)
    x = torch.randn(6, 1, 64)
    d = torch.tensor([3, -3, 7, -7, 1, -1])
    y = O.rotate(x, d, cos, sin)
    explicit = O.apply_rope(x, cos[d.abs()], sin[d.abs()] * torch.sign(d)[:, None].float())
    assert torch.equal(y, explicit)


# ---------------------------------------------------------- C oracle cross-checks
@pytest.mark.parametrize("dtype,code", [(torch.bfloat16, 0), (torch.float32, 2)])
def test_relocate_gather_python_equals_c_bit_exact(dtype, code):
    torch.manual_seed(4)
    L, S, H, D, T = 2, 40, 3, 64, 25
    cos, sin = O.rope_table(64, D)
    k = torch.randn(L, S, H, D).to(dtype)
    v = torch.randn(L, S, H, D).to(dtype)
    slot = torch.randint(0, S, (T,))
    delta = torch.randint(-40, 41, (T,))
    delta[::5] = 0
    pk, pv = O.relocate_rope_gather(k, v, slot, delta, cos, sin)
    npdt = np.uint16 if dtype == torch.bfloat16 else np.float32
    kn = _bits(k).numpy().view(npdt)
    vn = _bits(v).numpy().view(npdt)
    ck, cv = C.relocate_rope_gather(kn, vn, slot.numpy(), delta.numpy(), cos.numpy(), sin.numpy(), code)
    assert np.array_equal(_bits(pk).numpy().view(npdt), ck)
    assert np.array_equal(_bits(pv).numpy().view(npdt), cv)
    # delta == 0 rows are bit copies of the source rows
    z = delta == 0
    assert torch.equal(_bits(pk[:, z]), _bits(k[:, slot[z]]))


def test_reference_materialize_geometry_bit_exact_between_formulations():
    """Shapes of tests/test_attention_kernels.py:127-165 (L=2, 24 slots, Hkv=2, D=64, A=7, shift 5, dst 12)."""
    torch.manual_seed(0)
    L, S, H, D, A, shift, dst = 2, 24, 2, 64, 7, 5, 12
    k = torch.randn(L, S, H, D).to(torch.bfloat16)
    v = torch.randn_like(k)
    src_k, src_v = k[:, :A].clone(), v[:, :A].clone()
    cos, sin = O.rope_table(S, D)
    k2, v2 = k.clone(), v.clone()
    O.materialize_relocated_affix(k2, v2, cos, sin, dst, A, shift)
    expected = O.apply_rope(src_k.reshape(-1, H, D), cos[shift].expand(L * A, -1), sin[shift].expand(L * A, -1)).view_as(src_k)
    assert torch.equal(_bits(k2[:, dst:dst + A]), _bits(expected))
    assert torch.equal(_bits(v2[:, dst:dst + A]), _bits(src_v))
    # untouched elsewhere
    keep = torch.ones(S, dtype=torch.bool)
    keep[dst:dst + A] = False
    assert torch.equal(_bits(k2[:, keep]), _bits(k[:, keep]))
    # and equal to the gather form with slot = arange(A), delta = shift
    gk, gv = O.relocate_rope_gather(k, v, torch.arange(A), torch.full((A,), shift), cos, sin)
    assert torch.equal(_bits(gk), _bits(k2[:, dst:dst + A]))
    assert torch.equal(_bits(gv), _bits(v2[:, dst:dst + A]))


def test_scatter_then_gather_is_identity_and_minus_one_is_skipped():
    torch.manual_seed(5)
    S, H, D, N = 32, 2, 64, 12
    kc = torch.zeros(S, H, D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    key = torch.randn(N, H, D).to(torch.bfloat16)
    val = torch.randn(N, H, D).to(torch.bfloat16)
    slot = torch.randperm(S)[:N].to(torch.int32)
    slot[3] = -1
    O.store_kvcache(key, val, kc, vc, slot)
    live = slot >= 0
    gk, gv = O.relocate_rope_gather(kc[None], vc[None], slot[live], None, None, None)
    assert torch.equal(_bits(gk[0]), _bits(key[live]))
    assert torch.equal(_bits(gv[0]), _bits(val[live]))
    untouched = torch.ones(S, dtype=torch.bool)
    untouched[slot[live].long()] = False
    assert torch.all(kc[untouched] == 0) and torch.all(vc[untouched] == 0)
    # C restatement agrees bit for bit
    kc2 = np.zeros((S, H, D), np.uint16)
    vc2 = np.zeros((S, H, D), np.uint16)
    C.kv_scatter(kc2, vc2, _bits(key).numpy().view(np.uint16), _bits(val).numpy().view(np.uint16), slot.numpy(), 0)
    assert np.array_equal(kc2, _bits(kc).numpy().view(np.uint16))
    assert np.array_equal(vc2, _bits(vc).numpy().view(np.uint16))


# ----------------------------------------------------------------------- top-k
def test_topk_brute_force_on_tiny_inputs_with_ties():
    # every multiset of 5 scores drawn from 3 values, every k: enumerate the definition
    for scores in itertools.product([0.0, 1.0, 2.0], repeat=5):
        for k in range(6):
            for largest in (True, False):
                sign = -1 if largest else 1
                want = sorted(sorted(range(5), key=lambda i: (sign * scores[i], i))[:k])
                assert O.topk_anchors(torch.tensor(scores), k, largest) == want
                assert C.topk(np.array(scores, np.float32), k, largest).tolist() == want


def test_topk_matches_torch_when_boundary_is_untied_and_value_multiset_always():
    g = torch.Generator().manual_seed(6)
    for trial in range(30):
        A = int(torch.randint(5, 400, (1,), generator=g))
        s = torch.randn(A, generator=g).abs()
        if trial % 2:
            src = torch.randint(0, A, (max(A // 20, 1),), generator=g)
            dst = torch.randint(0, A, (max(A // 20, 1),), generator=g)
            s[dst] = s[src]
        k = O.anchor_budget(0.2, A)
        got = O.topk_anchors(s, k)
        vals, idx = torch.topk(s, k)
        assert sorted(s[got].tolist(), reverse=True) == sorted(vals.tolist(), reverse=True)
        srt = torch.sort(s, descending=True).values
        if k < A and srt[k - 1] != srt[k]:
            assert got == sorted(idx.tolist())
        assert got == sorted(got) and len(set(got)) == k
        assert C.topk(s.numpy(), k).tolist() == got


def test_topk_offsets_zero_and_full():
    s = torch.tensor([0.5, 0.5, 0.1, 0.9])
    assert O.topk_anchors(s, 0) == []
    assert O.topk_anchors(s, 4, offset=10) == [10, 11, 12, 13]
    assert O.topk_anchors(s, 9) == [0, 1, 2, 3]
    assert O.topk_anchors(s, 2) == [0, 3]
    assert O.topk_anchors(s, 2, largest=False) == [0, 2]
    assert O.topk_anchors(torch.tensor([0.0, -0.0, 1.0]), 2, largest=False) == [0, 1]


def test_anchor_budget_is_python_double_ceiling():
    assert O.anchor_budget(0.07, 100) == 8        # 0.07*100 = 7.000000000000001 in binary64
    assert O.anchor_budget(0.1, 30) == 3
    assert O.anchor_budget(0.2, 600) == 120
    assert O.anchor_budget(0.0, 600) == 0
    assert O.anchor_budget(1.0, 600) == 600
    assert O.anchor_budget(2.0, 7) == 7
    for r, a in [(0.05, 1000), (0.3, 999), (0.5, 1201), (0.07, 100)]:
        assert O.anchor_budget(r, a) == min(O.ceil_to_int(r * a), a) == min(math.ceil(r * a), a)


# -------------------------------------------------------------------- attention
@pytest.mark.parametrize("H,Hkv", [(4, 2), (4, 4), (6, 1)])
def test_dense_attention_matches_sdpa_and_c(H, Hkv):
    torch.manual_seed(7)
    Tq, Tk, D = 9, 23, 64
    q, k, v = torch.randn(Tq, H, D), torch.randn(Tk, Hkv, D), torch.randn(Tk, Hkv, D)
    got = O.dense_attention_reference(q, k, v, H, Hkv)
    g = H // Hkv
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(g, 0)[None],
        v.transpose(0, 1).repeat_interleave(g, 0)[None])[0].transpose(0, 1)
    torch.testing.assert_close(got, ref, atol=2e-6, rtol=1e-5)
    c = C.dense_attention(q.numpy(), k.numpy(), v.numpy(), D ** -0.5)
    np.testing.assert_allclose(got.numpy(), c, atol=2e-6, rtol=1e-5)


def test_attention_invariants():
    torch.manual_seed(8)
    H, Hkv, D = 4, 2, 64
    kc = torch.randn(4, 8, Hkv, D)
    vc = torch.randn(4, 8, Hkv, D)
    q = torch.randn(5, H, D)
    slots = torch.randperm(32)[:13].to(torch.int32)
    cu_q, cu_k = torch.tensor([0, 5]), torch.tensor([0, 13])
    out = O.acache_attention(q, kc, vc, cu_q, cu_k, slots)
    # permuting a request's keys leaves the output unchanged
    perm = torch.randperm(13)
    out_p = O.acache_attention(q, kc, vc, cu_q, cu_k, slots[perm])
    torch.testing.assert_close(out, out_p, atol=1e-5, rtol=1e-5)
    # all-equal V rows -> every output row is that row
    vconst = torch.ones_like(vc) * torch.randn(1, 1, Hkv, D)
    out_c = O.acache_attention(q, kc, vconst, cu_q, cu_k, slots)
    torch.testing.assert_close(out_c, vconst[0, 0].repeat_interleave(2, 0)[None].expand(5, -1, -1), atol=1e-5, rtol=1e-5)
    # a duplicated request gives duplicated outputs; an empty request gives zeros
    out2 = O.acache_attention(torch.cat([q, q]), kc, vc, torch.tensor([0, 5, 10, 10]), torch.tensor([0, 13, 26, 26]),
                              torch.cat([slots, slots]))
    assert torch.equal(out2[:5], out2[5:]) and torch.equal(out2[:5], out)
    out3 = O.acache_attention(q, kc, vc, torch.tensor([0, 5]), torch.tensor([0, 0]), slots[:0])
    assert torch.all(out3 == 0)


def test_relocation_modes_are_equivalent():
    """key side == plain attention over materialised keys == query side (shared keys packed first)."""
    torch.manual_seed(9)
    H, Hkv, D = 4, 2, 64
    S = 64
    A, a0 = 5, 7          # affix of 5 shared rows placed at logical position 7
    kv_len, q_len = 17, 6
    kc = torch.randn(S, Hkv, D).to(torch.bfloat16)
    vc = torch.randn(S, Hkv, D).to(torch.bfloat16)
    q = torch.randn(q_len, H, D).to(torch.bfloat16)
    cos, sin = O.rope_table(S, D)
    read = list(range(A, A + kv_len))
    for local, pos in enumerate(range(a0, a0 + A)):
        read[pos] = local
    cu_q, cu_k = torch.tensor([0, q_len]), torch.tensor([0, kv_len])
    shifts = torch.tensor([a0])
    key_side = O.acache_attention(q, kc, vc, cu_q, cu_k, torch.tensor(read), shared_prefix_len=A,
                                  affix_shifts=shifts, rope_cos=cos, rope_sin=sin)
    # materialise the rotated copy at slots 40.. and read it with plain attention
    kc2, vc2 = kc.clone()[None], vc.clone()[None]
    O.materialize_relocated_affix(kc2, vc2, cos, sin, 40, A, a0)
    read_m = list(read)
    for local, pos in enumerate(range(a0, a0 + A)):
        read_m[pos] = 40 + local
    mat = O.acache_attention(q, kc2[0], vc2[0], cu_q, cu_k, torch.tensor(read_m))
    assert torch.equal(mat, key_side)
    # query side over the packed layout
    packed, shared_len = O.attention_read_layout(read, 0, A, a0, True)
    assert shared_len == A
    qs = O.acache_attention(q, kc, vc, cu_q, cu_k, torch.tensor(packed), shared_prefix_len=A,
                            shared_kv_lens=torch.tensor([shared_len]), affix_shifts=shifts, rope_cos=cos, rope_sin=sin)
    torch.testing.assert_close(qs.float(), key_side.float(), atol=5e-2, rtol=5e-2)
    # and all of them equal attention over keys rotated in float64-free closed form
    deltas = torch.tensor(O.key_side_deltas(read, A))
    assert deltas.tolist() == [0] * a0 + [a0] * A + [0] * (kv_len - a0 - A)


# -------------------------------------------------- golden vectors of the reference
def test_attention_read_layout_golden_vectors():
    """tests/test_model_runner_acache.py:26-47."""
    read = [8, 9, 0, 10, 2, 11]
    assert O.attention_read_layout(read, 0, 3, 2, True) == ([0, 2, 8, 9, 10, 11], 2)
    assert O.attention_read_layout(read, 0, 3, 2, False) == ([8, 9, 0, 10, 2, 11], 0)
    assert O.attention_read_layout(read, 0, 3, 0, True) == (read, 0)


@pytest.mark.parametrize(
    "num_tokens,a0,a1,gen_start",
    [(5, 0, 2, 3), (6, 1, 3, 4), (5, 3, 5, 1)],  # the three span layouts of tests/test_sequence_spans.py:11-45
)
def test_finalize_slot_mapping_reference_assertions(num_tokens, a0, a1, gen_start):
    A = a1 - a0
    K = O.anchor_budget(0.5, A)
    anchor = a1 - 1
    nblocks = -(-(K + num_tokens - A) // 4)
    table = list(range(2, 2 + nblocks))
    read, rpos, rslots = O.finalize_slot_mapping(num_tokens, a0, a1, [anchor], table, 4, 0)
    non_affix = list(range(a0)) + list(range(a1, num_tokens))
    assert rpos == sorted([anchor] + non_affix)
    assert read[a0] == 0
    assert read[anchor] != anchor - a0
    assert all(s >= 0 for s in read)
    assert rpos.index(gen_start) >= 0
    # anchors take the first private slots, the rest follow in position order
    priv = O.private_slots(table, K + num_tokens - A, 4)
    assert read[anchor] == priv[0]
    assert [read[p] for p in non_affix] == priv[K:]
    assert rslots == [read[p] for p in rpos]


def test_get_transfer_index_closed_form():
    logits = torch.tensor([[[5.0, 0.0, 0.0, 0.0], [1.0, 1.0, 1.0, 1.0], [2.0, 1.0, 1.0, 1.0]]])
    mask = torch.tensor([[True, True, True]])
    x = torch.full((1, 3), 9)
    x0, t = O.get_transfer_index(logits, mask, x, threshold=0.9)
    assert x0.tolist() == [[0, 0, 0]]
    assert t.tolist() == [[True, False, False]]      # softmax(5,0,0,0)[0] = 0.98 >= 0.9
    x0, t = O.get_transfer_index(logits, torch.tensor([[False, True, True]]), x, threshold=0.9)
    assert x0.tolist() == [[9, 0, 0]]
    assert t.tolist() == [[False, False, True]]      # nothing reaches 0.9: force the most confident masked row


# ------------------------------------------------------------------ affix importance (model_runner.py:730-773)
def test_affix_importance_closed_forms_and_brute_force():
    g = torch.Generator().manual_seed(11)
    H, Hkv, D, A, S = 4, 2, 64, 9, 16
    cos, sin = O.rope_table(64, D, 1e4)
    kc = torch.randn(S, Hkv, D, generator=g).to(torch.bfloat16)
    q = torch.randn(12, H, D, generator=g).to(torch.bfloat16)
    mask_rows = torch.tensor([1, 4, 5, 7, 8, 9, 10], dtype=torch.int32)
    cu = torch.tensor([0, 3, 3, 7], dtype=torch.int32)            # request 1 has no [MASK] query
    shifts = torch.tensor([0, 5, 11], dtype=torch.int32)
    imp = O.affix_importance(q, kc, mask_rows, cu, A, affix_shifts=shifts, cos=cos, sin=sin, affix_slot0=2)
    assert imp.shape == (3, A)
    # every softmax row sums to one: the total is (mask rows) x (heads)
    assert torch.allclose(imp.sum(1), torch.tensor([3.0 * H, 0.0, 4.0 * H]), atol=1e-4)
    # brute force of the definition, request 2 (shift 11)
    kr = O.rotate(kc[2:2 + A], torch.full((A,), 11, dtype=torch.int32), cos, sin).float()
    want = torch.zeros(A)
    for r in mask_rows[3:7].tolist():
        for h in range(H):
            s = torch.tensor([float(q[r, h].float() @ kr[a, h // 2]) for a in range(A)]) * D ** -0.5
            want += torch.softmax(s, 0)
    assert torch.allclose(imp[2], want, atol=1e-4)
    # identical keys: every affix token gets the same share
    same = kc.clone()
    same[:] = kc[0]
    u = O.affix_importance(q, same, mask_rows, cu, A)
    assert torch.allclose(u[0], torch.full((A,), 3.0 * H / A), atol=1e-5)


# ------------------------------------------------------------------ fused rotary + scatter (modeling_llada.py:412-453, attention.py:22-41)
def test_rope_qk_scatter_is_rotation_at_positions_then_scatter():
    g = torch.Generator().manual_seed(5)
    N, H, Hkv, D = 7, 4, 2, 64
    cos, sin = O.rope_table(32, D, 1e4)
    q = torch.randn(N, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(N, Hkv, D, generator=g, dtype=torch.float64)
    v = torch.randn(N, Hkv, D, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 3, 3, 31, 7, 1, 20])
    slots = torch.tensor([5, -1, 0, 9, 2, -1, 7], dtype=torch.int32)
    kc = torch.full((12, Hkv, D), 7.0, dtype=torch.float64)
    vc = torch.full((12, Hkv, D), 7.0, dtype=torch.float64)
    q_rot, k_rot = O.rope_qk_scatter(q, k, v, pos, cos.double(), sin.double(), kc, vc, slots)
    # explicit 2x2 rotation of every (d, d + D/2) pair by pos * theta^(-2d/D), in float64
    inv = 1e4 ** (-torch.arange(0, D, 2, dtype=torch.float64) / D)
    ang = pos.double()[:, None] * inv[None, :]
    for x, y in ((q, q_rot), (k, k_rot)):
        lo, hi = x[..., :D // 2], x[..., D // 2:]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        want = torch.cat((lo * c - hi * s, hi * c + lo * s), dim=-1)
        assert torch.allclose(y, want, atol=1e-6)          # the tables are fp32
    assert torch.equal(q_rot[0], q[0]) and torch.equal(k_rot[0], k[0])   # position 0: identity
    # the cache holds the rotated k and the plain v at the mapped slots, nothing else moved
    for i, s in enumerate(slots.tolist()):
        if s >= 0:
            assert torch.equal(kc[s], k_rot[i]) and torch.equal(vc[s], v[i])
    untouched = [s for s in range(12) if s not in slots.tolist()]
    assert (kc[untouched] == 7.0).all() and (vc[untouched] == 7.0).all()
    # without a slot map nothing is written
    kc2 = kc.clone()
    O.rope_qk_scatter(q, k, v, pos, cos.double(), sin.double(), kc2, vc, None)
    assert torch.equal(kc2, kc)


# ------------------------------------------------------------------ token and confidence (model_runner.py:2279-2296)
def test_argmax_confidence_against_float64_softmax_and_edge_rows():
    g = torch.Generator().manual_seed(6)
    logits = (torch.randn(5, 3, 97, generator=g) * 4).to(torch.bfloat16)
    tok, conf = O.argmax_confidence(logits)
    p = torch.softmax(logits.double(), dim=-1)
    assert tok.shape == conf.shape == (5, 3)
    assert torch.equal(tok, p.argmax(-1))
    assert torch.allclose(conf.double(), p.max(-1).values, rtol=1e-5)
    # given picks: their probability, the picks handed back
    picks = torch.randint(0, 97, (5, 3), generator=g)
    tok2, conf2 = O.argmax_confidence(logits, picks)
    assert torch.equal(tok2, picks)
    assert torch.allclose(conf2.double(), p.gather(-1, picks[..., None]).squeeze(-1), rtol=1e-5)
    # ties go to the first maximum; a one-hot row has confidence 1; a uniform row 1/V
    rows = torch.zeros(3, 8)
    rows[0, 2] = rows[0, 5] = 3.0
    rows[1, 6] = 200.0
    tok3, conf3 = O.argmax_confidence(rows)
    assert tok3.tolist() == [2, 6, 0]
    assert abs(float(conf3[1]) - 1.0) < 1e-6 and abs(float(conf3[2]) - 1 / 8) < 1e-7
    assert abs(float(conf3[0]) - math.exp(3) / (2 * math.exp(3) + 6)) < 1e-6
