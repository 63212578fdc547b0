"""The life of a request on real pools, one GatedDeltaNet layer, two sequences: chunked prefill -> admission into a slot
(Pools.load) -> batched decode steps -> plain to speculative (to_spec) -> a verify round of M tokens -> commit of the accepted
prefix (to_plain) -> decode again.  The chain exercises the conventions that tie the operators together (the conv buffer a
step reads is `pos & 1`, a verify round reads buffer `par` and writes the other, snapshot j is the state after token j) and
is checked against the sequential float64 restatement of the layer core over the accepted tokens (qwen35/batch.py:431-447,
qwen35/serve.py:310-348, qwen35/batch_spec.py:45-150)."""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
PW, CD = 8224, 6144


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    return q


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


def test_prefill_admission_decode_verify_commit_chain(qt, dev):
    from qwen_tailor_amd.model import Cfg
    M, D1, D2 = 4, 5, 3
    T0 = [150, 67]                     # prompt lengths (neither a multiple of the chunk; odd and even positions after them)
    accepted = [3, 1]                  # tokens of the verify round that each sequence keeps
    slots = [1, 0]
    gen = torch.Generator().manual_seed(4242)
    cw, A_log, dtb, gw = layer_params(4242)
    rows = [rand_bf(gen, (T0[b] + D1 + M + D2, PW), 1.0) for b in range(2)]
    cs0 = [rand_bf(gen, (3, CD)) for _ in range(2)]
    S0 = [(torch.randn((16, 128, 128), generator=gen) * 0.02).numpy() for _ in range(2)]
    dcw, dA, ddt, dgw = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev)

    cfg = Cfg(layers=4)                # three GatedDeltaNet layers and one attention layer; layer 0 is the one driven here
    P = qt.batch.Pools(cfg, 3, 256, device=dev)
    SP = qt.batch_spec.SpecPools(cfg, 2, 3, M, 256, device=dev)
    got = [[], []]                     # gated outputs per sequence, in token order

    # prefill and admission
    pos = list(T0)
    for b in range(2):
        out, conv1, ssm1 = qt.prefill.gdn_core(to_dev(rows[b][:T0[b]], dev, BF16), to_dev(cs0[b][None], dev, BF16),
                                               to_dev(S0[b][None], dev), dcw, dA, ddt, dgw)
        got[b].append(to_np(out))
        P.load(slots[b], {"conv": [conv1], "ssm": [ssm1], "kv": []}, pos[b])
    dslots = to_dev(np.array(slots, np.int32), dev)

    def decode(n):
        for _ in range(n):
            step = to_dev(np.stack([rows[b][pos[b]] for b in range(2)]), dev, BF16)
            y = qt.batch.deltanet_b(step, P.conv[0], dcw, dA, ddt, P.ssm[0], dslots, to_dev(np.array(pos, np.int32), dev))
            o = to_np(qt.batch.gnorm_rows(y, step, dgw))
            for b in range(2):
                got[b].append(o[b:b + 1])
                pos[b] += 1

    decode(D1)
    # plain -> speculative, one verify round, commit of the accepted prefix
    for b in range(2):
        qt.batch_spec.to_spec(P, SP, slots[b], pos[b], b)
    vrows = to_dev(np.concatenate([rows[b][pos[b]:pos[b] + M] for b in range(2)]), dev, BF16)
    zeros = to_dev(np.zeros(2, np.int32), dev)
    y = qt.batch_spec.deltanet_bm(vrows, SP.conv[0], dcw, dA, ddt, SP.ssm[0], to_dev(np.array([0, 1], np.int32), dev), zeros, zeros, M)
    o = to_np(qt.batch.gnorm_rows(y, vrows, dgw))
    keep = []                          # rows of each sequence that make up its accepted history
    for b in range(2):
        a = accepted[b]
        got[b].append(o[b * M:b * M + a])
        keep.append(list(range(pos[b] + a)))
        pos[b] += a
        qt.batch_spec.to_plain(P, SP, slots[b], pos[b], b, 1, a - 1)      # the round read buffer 0 and wrote buffer 1
    # the rejected draft tokens are dropped; the next real tokens are the rows after the verify block
    nxt = [T0[b] + D1 + M for b in range(2)]
    for b in range(2):
        keep[b] += list(range(nxt[b], nxt[b] + D2))
    for _ in range(D2):
        step = to_dev(np.stack([rows[b][nxt[b]] for b in range(2)]), dev, BF16)
        yy = qt.batch.deltanet_b(step, P.conv[0], dcw, dA, ddt, P.ssm[0], dslots, to_dev(np.array(pos, np.int32), dev))
        oo = to_np(qt.batch.gnorm_rows(yy, step, dgw))
        for b in range(2):
            got[b].append(oo[b:b + 1])
            pos[b] += 1
            nxt[b] += 1

    for b in range(2):
        hist = rows[b][keep[b]]
        want, _, tail, state = O.prefill_gdn(hist, cs0[b], cw, A_log, dtb, S0[b], gw)
        out = np.concatenate(got[b])
        assert out.shape == want.shape, (out.shape, want.shape)
        check_rel(f"sequence {b}: prompt outputs", out[:T0[b]], want[:T0[b]], 2e-3, rel_l2)
        check_rel(f"sequence {b}: decode / verify outputs", out[T0[b]:], want[T0[b]:], 2e-3, rel_l2)
        st = P.read(slots[b], pos[b])
        check_rel(f"sequence {b}: final state", to_np(st["ssm"][0])[0], state, 2e-3, rel_l2)
        check_equal(f"sequence {b}: conv window", to_np(st["conv"][0])[0], tail)
    # the third slot, the trash slot and the layers that were not driven stay zero
    assert float(P.ssm[0][2].abs().max()) == 0.0 and float(P.ssm[1].abs().max()) == 0.0 and float(P.conv[2].abs().max()) == 0.0


def test_attention_prefill_admission_decode_verify_chain(qt, dev):
    """One full-attention layer between its qkv projection and its output gate: causal prefill over the prompt -> the prompt's
    K / V rows admitted into a slot (Pools.load) -> decode rows that append their keys -> a verify round of M rows; every output
    row against the float64 causal attention over the whole history (qwen35/model.py:154-169, qwen35/batch.py:141-237, 431-447)."""
    from qwen_tailor_amd.model import Cfg
    S, D, M, Lmax, slot = 203, 3, 4, 256, 2
    T = S + D + M
    rng = np.random.default_rng(515)
    qkv = bf(rng.standard_normal((T, O.QKV_W)))
    qn, kn = bf(1 + 0.1 * rng.standard_normal(256)), bf(1 + 0.1 * rng.standard_normal(256))
    dqkv, dqn, dkn = to_dev(qkv, dev, BF16), to_dev(qn, dev, BF16), to_dev(kn, dev, BF16)
    # the oracle's whole history at once
    oq, ok, ov = O.attn_qkv_prep(qkv, qn, kn, np.zeros(1, np.int32), T)             # one sequence of T rows: positions 0 .. T-1
    ref = O.sdpa_causal(oq.transpose(1, 0, 2), ok.transpose(1, 0, 2), ov.transpose(1, 0, 2))      # [8, T, 256]
    want = O.attn_out_gate(bf(ref.transpose(1, 0, 2)), qkv)
    # prefill: rows 0 .. S-1
    q, k, v = qt.attention.qkv_prep(dqkv[:S], dqn, dkn, to_dev(np.zeros(1, np.int32), dev), S)
    Kc = torch.zeros((1, 2, Lmax, 256), dtype=BF16, device=dev)
    Vc = torch.zeros((1, 2, Lmax, 256), dtype=BF16, device=dev)
    Kc[0, :, :S], Vc[0, :, :S] = k.transpose(0, 1), v.transpose(0, 1)
    o = qt.attention.scaled_dot_product_attention(q.transpose(0, 1)[None].contiguous(), Kc[:, :, :S], Vc[:, :, :S], scale=256 ** -0.5,
                                                  mask="causal")
    got = [to_np(qt.attention.out_gate(o[0].transpose(0, 1).contiguous(), dqkv[:S]))]
    cfg = Cfg(layers=4)
    P = qt.batch.Pools(cfg, 3, Lmax, device=dev)
    P.load(slot, {"conv": [], "ssm": [], "kv": [(Kc, Vc)]}, S)
    dslot = to_dev(np.array([slot], np.int32), dev)
    pos = S
    for rows in [1] * D + [M]:                                   # decode rows one by one, then a verify round of M rows
        dpos = to_dev(np.array([pos], np.int32), dev)
        q, k, v = qt.attention.qkv_prep(dqkv[pos:pos + rows], dqn, dkn, dpos, rows)
        o = qt.batch.attn_b(q, k, v, P.K[0], P.V[0], dslot, dpos, M=rows)
        got.append(to_np(qt.attention.out_gate(o, dqkv[pos:pos + rows])))
        pos += rows
    out = np.concatenate(got)
    assert out.shape == want.shape
    check_rel("prompt rows", out[:S], want[:S], 1e-2, rel_l2)
    for r in range(S, T):
        check_rel(f"row {r}", out[r], want[r], 1e-2, rel_l2)
    check_equal("keys in the pool", to_np(P.K[0][slot, :, :T]), ok.transpose(1, 0, 2))
    check_equal("values in the pool", to_np(P.V[0][slot, :, :T]), ov.transpose(1, 0, 2))
    assert float(P.K[0][0].abs().max()) == 0.0 and float(P.K[0][3].abs().max()) == 0.0          # other slots and the trash slot


@pytest.mark.parametrize("T1,T2", [(150, 100), (64, 7), (33, 300)])
def test_prefill_resumed_from_a_checkpoint_equals_one_prefill(qt, dev, T1, T2):
    """A prompt prefilled in two pieces, the second starting from the first's state as a prefix-cache hit would (conv window and
    recurrent state carried over): same outputs and final state as one prefill of the whole prompt, within the chunked form's
    tolerance (the chunk borders differ), the conv window bit for bit; both against the sequential float64 restatement."""
    gen = torch.Generator().manual_seed(T1 * 1000 + T2)
    cw, A_log, dtb, gw = layer_params(T1 + T2)
    rows = rand_bf(gen, (T1 + T2, PW), 1.0)
    cs0 = rand_bf(gen, (3, CD))
    S0 = (torch.randn((16, 128, 128), generator=gen) * 0.02).numpy()
    dcw, dA, ddt, dgw = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev)
    drows = to_dev(rows, dev, BF16)
    whole, conv_w, ssm_w = qt.prefill.gdn_core(drows, to_dev(cs0[None], dev, BF16), to_dev(S0[None], dev), dcw, dA, ddt, dgw)
    o1, conv1, ssm1 = qt.prefill.gdn_core(drows[:T1], to_dev(cs0[None], dev, BF16), to_dev(S0[None], dev), dcw, dA, ddt, dgw)
    o2, conv2, ssm2 = qt.prefill.gdn_core(drows[T1:], conv1, ssm1, dcw, dA, ddt, dgw)
    want, _, tail, state = O.prefill_gdn(rows, cs0, cw, A_log, dtb, S0, gw)
    pieces = np.concatenate([to_np(o1), to_np(o2)])
    check_rel("two pieces against one prefill", pieces, to_np(whole), 2e-3, rel_l2)
    check_rel("two pieces against the restatement", pieces, want, 2e-3, rel_l2)
    check_rel("final state against one prefill", to_np(ssm2), to_np(ssm_w), 2e-3, rel_l2)
    check_rel("final state against the restatement", to_np(ssm2)[0], state, 2e-3, rel_l2)
    check_tensors_equal("conv window", conv2, conv_w)
    check_equal("conv window against the restatement", to_np(conv2)[0], tail)
