"""Pins oracle/policy_loop.py (the restatement of the FSDP trainer's micro-batch loops,
policy_trainer.py:80-172, 203-311, 316-365) with a three-sample case worked by hand.

Every expected table below is a literal derived on paper from the reference lines, not from
the oracle's own helpers, so that a shared misreading of the label roll, the mask shift, the
packing order or the record slicing fails here.

The case: vocabulary 7; three samples
    s0: prompt 2 + response 3, tokens [1,2,3,4,5]
    s1: prompt 1 + response 2, tokens [6,1,2]
    s2: prompt 1 + response 1, tokens [3,4]
The toy model returns logits[b,s,:] = log P[token[b,s]] with P[tok][v] = q[(v - tok) mod 7],
q = (1/2, 1/4, 1/8, 1/16, 1/32, 1/64, 1/64).  So log-softmax(logits)[v] = log q[(v-tok) mod 7]
exactly, and every row has entropy (1/2*1 + 1/4*2 + 1/8*3 + 1/16*4 + 1/32*5 + 2/64*6) ln 2
= 1.96875 ln 2.
"""
import math

import pytest
import torch

from oracle import policy_loop as opl

LN2 = math.log(2.0)
Q_EXP = [1, 2, 3, 4, 5, 6, 6]            # q[j] = 2 ** -Q_EXP[j]
ENTROPY = 1.96875 * LN2


def lp_of(tok, label):
    """log P[tok][label], by hand: -ln2 * exponent of q[(label - tok) mod 7]."""
    return -LN2 * Q_EXP[(label - tok) % 7]


class ToyModel(torch.nn.Module):
    """logits = table[token]; the table is a parameter so that gradients can be checked."""

    def __init__(self):
        super().__init__()
        q = torch.tensor([2.0 ** -e for e in Q_EXP], dtype=torch.float64)
        rows = [torch.roll(q, shifts=tok) for tok in range(7)]     # P[tok][v] = q[(v - tok) mod 7]
        self.table = torch.nn.Parameter(torch.log(torch.stack(rows)))
        self.calls = []

    def forward(self, input_ids, position_ids):
        self.calls.append((input_ids.clone(), position_ids.clone()))
        return self.table[input_ids]


def samples(training):
    toks = [[1, 2, 3, 4, 5], [6, 1, 2], [3, 4]]
    p = [2, 1, 1]
    r = [3, 2, 1]
    out = []
    for i in range(3):
        d = {"all_tokens": torch.tensor(toks[i]), "prompt_token_length": p[i], "response_token_length": r[i]}
        if training:
            # per-position logprobs of the label each position predicts inside its own padded row
            # (what forward_step stores: length p + r)
            d["old_logprobs"] = torch.tensor(OLD[i], dtype=torch.float64)
            d["ref_logprobs"] = torch.tensor(REF[i], dtype=torch.float64)
            d["advantages"] = ADV[i]
        out.append(d)
    return out


# ---- hand-worked tables -------------------------------------------------------------------------
# Padded layout, micro-batch size 3 (one micro-batch, S = 5):
#   tokens  [[1,2,3,4,5],[6,1,2,0,0],[3,4,0,0,0]]
#   labels = roll(tokens, -1, dim 1)      (policy_trainer.py:135)
PADDED_LABELS = [[2, 3, 4, 5, 1], [1, 2, 0, 0, 6], [4, 0, 0, 0, 3]]
#   attention mask [i, :p+r] = 1, loss mask [i, p:p+r] = 1   (trainer_utils.py:60-96)
PADDED_ATTN = [[1, 1, 1, 1, 1], [1, 1, 1, 0, 0], [1, 1, 0, 0, 0]]
#   training mask = roll(loss_mask, -1) with the last column zeroed (policy_trainer.py:160-162):
#   loss mask [[0,0,1,1,1],[0,1,1,0,0],[0,1,0,0,0]] ->
PADDED_TRAIN_MASK = [[0, 1, 1, 1, 0], [1, 1, 0, 0, 0], [1, 0, 0, 0, 0]]

# Packing with max_token_in_seq = 6 (packing_utils.py:23-83,105-148): lengths [5,3,2]
#   bin_packing: 5 -> bin0; 3: bin0 has 1 left, not > 3 -> bin1; 2: bin0 no, bin1 has 3 > 2 -> bin1  => 2 bins
#   bin_packing_fix_bin(2): 5 -> bin0; 3 -> bin1; 2 -> bin1 (3+2 < 5+2); totals tie 5 = 5, so the
#   descending sort compares the id lists: [1,2] > [0]  =>  micro-batches [[s1,s2],[s0]]
PACKED_SAMPLE_IDS = [[1, 2], [0]]
#   micro-batch 0: padded [[6,1,2],[3,4,0]] (S=3), attn [[1,1,1],[1,1,0]] -> packed row, flat indices, position ids
PACKED_TOKENS = [[6, 1, 2, 3, 4], [1, 2, 3, 4, 5]]
PACKED_INDICES = [[0, 1, 2, 3, 4], [0, 1, 2, 3, 4]]
PACKED_POSITIONS = [[0, 1, 2, 0, 1], [0, 1, 2, 3, 4]]
#   labels roll along the PACKED row: the last position of s1 predicts s2's first token
PACKED_LABELS = [[1, 2, 3, 4, 6], [2, 3, 4, 5, 1]]
#   training masks stay in the padded [B,S] layout: loss masks [[0,1,1],[0,1,0]] and [[0,0,1,1,1]] ->
PACKED_TRAIN_MASK = [[[1, 1, 0], [1, 0, 0]], [[0, 1, 1, 1, 0]]]
N_RESPONSE_TOKENS = 6.0                      # 3 + 2 + 1 (policy_trainer.py:82)

# Per-sample logprob records (policy_trainer.py:343-363): position t of a sample holds
# log P[token_t][label_t]; the label of a sample's last position is the roll's wrap-around:
#   padded:  s0 labels [2,3,4,5,1], s1 [1,2,0] (third label is the pad 0), s2 [4,0]
#   packed:  s0 alone in its micro-batch: [2,3,4,5,1]; s1 [1,2,3] (next sequence's first token); s2 [4,6] (wrap)
RECORD_LABELS_PADDED = [[2, 3, 4, 5, 1], [1, 2, 0], [4, 0]]
RECORD_LABELS_PACKED = [[2, 3, 4, 5, 1], [1, 2, 3], [4, 6]]
TOKENS = [[1, 2, 3, 4, 5], [6, 1, 2], [3, 4]]

# Training inputs: old = lp - ln(ratio) with hand-picked ratios per position, ref = lp - 0.1 at
# every position (k = ref - lp = -0.1), advantages [+2, -1, +0.5] (Python floats -> fp32 column,
# promoted to the float64 of the logprobs in the product -A * ratio).
LP_PADDED = [[lp_of(t, l) for t, l in zip(TOKENS[i], RECORD_LABELS_PADDED[i])] for i in range(3)]
RATIO = [[1.0, 1.1, 1.5, 0.5, 1.0], [0.7, 1.0, 1.0], [1.3, 1.0]]
OLD = [[lp - math.log(rt) for lp, rt in zip(LP_PADDED[i], RATIO[i])] for i in range(3)]
REF = [[lp - 0.1 for lp in LP_PADDED[i]] for i in range(3)]
ADV = [2.0, -1.0, 0.5]
# Masked positions (padded training mask rows above): s0 positions 1,2,3; s1 positions 0,1; s2 position 0.
# Surrogate by hand, clip range [0.8, 1.2], final clip 3 (loss_gallery.py:6-33), L = max(-A r, -A clamp(r)):
#   s0 A=+2:  r=1.1 -> -2.2;  r=1.5 -> max(-3.0, -2.4) = -2.4;  r=0.5 -> max(-1.0, -1.6) = -1.0
#   s1 A=-1:  r=0.7 -> max(0.7, 0.8) = 0.8;  r=1.0 -> 1.0
#   s2 A=+.5: r=1.3 -> max(-0.65, -0.6) = -0.6
PG_TOKENS = [-2.2, -2.4, -1.0, 0.8, 1.0, -0.6]
PG_LOSS = sum(PG_TOKENS) / N_RESPONSE_TOKENS
KL_TOKEN = math.exp(-0.1) + 0.1 - 1.0        # k3 estimator at k = -0.1 (policy_trainer.py:268-276)


def test_preprocess_padded_tables():
    n, mbs = opl.preprocess_data_list(samples(True), True, packing=False, train_micro_batch_size=3)
    assert float(n) == N_RESPONSE_TOKENS and len(mbs) == 1
    mb = mbs[0]
    assert mb["all_tokens"].tolist() == [[1, 2, 3, 4, 5], [6, 1, 2, 0, 0], [3, 4, 0, 0, 0]]
    assert mb["labels"].tolist() == PADDED_LABELS
    assert mb["attention_mask"].tolist() == PADDED_ATTN
    assert mb["loss_mask"].tolist() == PADDED_TRAIN_MASK
    assert mb["position_ids"].tolist() == [[0, 1, 2, 3, 4]] * 3
    assert mb["sample_ids"] == [0, 1, 2] and mb["indices"] is None
    assert (mb["ori_batch_size"], mb["ori_seq_len"], mb["pad_size"]) == (3, 5, 0)
    # micro-batch size 2: ceil(3/2) micro-batches in list order (trainer_utils.py:110-123)
    _, two = opl.preprocess_data_list(samples(True), True, packing=False, train_micro_batch_size=2)
    assert [m["sample_ids"] for m in two] == [[0, 1], [2]]
    assert two[1]["labels"].tolist() == [[4, 3]] and two[1]["loss_mask"].tolist() == [[1, 0]]
    # without training the generate micro-batch size applies and no training fields are attached
    _, gen = opl.preprocess_data_list(samples(False), False, packing=False, generate_micro_batch_size=1)
    assert [m["sample_ids"] for m in gen] == [[0], [1], [2]] and "loss_mask" not in gen[0]


def test_preprocess_packed_tables():
    n, mbs = opl.preprocess_data_list(samples(True), True, packing=True, max_token_in_seq=6)
    assert float(n) == N_RESPONSE_TOKENS
    assert [m["sample_ids"] for m in mbs] == PACKED_SAMPLE_IDS
    for k, mb in enumerate(mbs):
        assert mb["all_tokens"].tolist() == [PACKED_TOKENS[k]]
        assert mb["indices"].tolist() == PACKED_INDICES[k]
        assert mb["position_ids"].tolist() == [PACKED_POSITIONS[k]]
        assert mb["labels"].tolist() == [PACKED_LABELS[k]]
        assert mb["loss_mask"].tolist() == PACKED_TRAIN_MASK[k]
    assert (mbs[0]["ori_batch_size"], mbs[0]["ori_seq_len"]) == (2, 3)
    assert (mbs[1]["ori_batch_size"], mbs[1]["ori_seq_len"]) == (1, 5)
    # a cap that holds everything: one bin, list order kept, indices skip the padding of the [3,5] layout
    _, one = opl.preprocess_data_list(samples(True), True, packing=True, max_token_in_seq=11)
    assert [m["sample_ids"] for m in one] == [[0, 1, 2]]
    assert one[0]["all_tokens"].tolist() == [[1, 2, 3, 4, 5, 6, 1, 2, 3, 4]]
    assert one[0]["indices"].tolist() == [0, 1, 2, 3, 4, 5, 6, 7, 10, 11]
    assert one[0]["labels"].tolist() == [[2, 3, 4, 5, 6, 1, 2, 3, 4, 1]]
    assert one[0]["position_ids"].tolist() == [[0, 1, 2, 3, 4, 0, 1, 2, 0, 1]]


@pytest.mark.parametrize("packing", [False, True])
def test_forward_step_records(packing):
    model = ToyModel()
    data = samples(False)
    kw = dict(max_token_in_seq=6) if packing else dict(generate_micro_batch_size=3)
    out = opl.forward_step(model, data, packing=packing, trainable=True, **kw)
    labels = RECORD_LABELS_PACKED if packing else RECORD_LABELS_PADDED
    for i in range(3):
        rec = out[i]["old_logprobs"]
        assert rec.shape == (len(TOKENS[i]),)                 # prompt + response positions (policy_trainer.py:361-363)
        want = [lp_of(t, l) for t, l in zip(TOKENS[i], labels[i])]
        assert rec.tolist() == pytest.approx(want, abs=1e-12)
        assert "ref_logprobs" not in out[i]
    # the model saw the packed rows / the padded batch, with the position ids of the tables above
    if packing:
        assert [c[0].tolist() for c in model.calls] == [[PACKED_TOKENS[0]], [PACKED_TOKENS[1]]]
        assert [c[1].tolist() for c in model.calls] == [[PACKED_POSITIONS[0]], [PACKED_POSITIONS[1]]]
    ref = opl.forward_step(ToyModel(), samples(False), packing=packing, trainable=False, **kw)
    assert "ref_logprobs" in ref[0] and "old_logprobs" not in ref[0]


@pytest.mark.parametrize("packing", [False, True])
def test_train_step_stats_and_gradient(packing):
    """Masked positions are the same in both layouts (none of them is a sequence's last position, where
    the packed label differs), so the hand-worked stats hold for both."""
    model = ToyModel()
    kw = dict(max_token_in_seq=6) if packing else dict(train_micro_batch_size=3)
    args = {"entropy_coef": 0.01, "kl_coef": 0.05}
    stats, totals = opl.train_step(model, samples(True), packing=packing, module_args=args, **kw)
    assert stats["pg_loss"] == pytest.approx(PG_LOSS, rel=1e-6)           # sum over masked tokens / N   (:301)
    assert stats["kl_loss"] == pytest.approx(KL_TOKEN, rel=1e-6)           # plain mean over masked tokens (:302)
    assert stats["entropy_loss"] == pytest.approx(ENTROPY, rel=1e-6)       # plain mean (:303); the chunked entropy buffer is fp32 (trainer_utils.py:38)
    # total = pg - entropy_coef * sum(H)/N + kl_coef * sum(kl)/N, summed over the micro-batches (:278-286)
    want_total = PG_LOSS - 0.01 * ENTROPY + 0.05 * KL_TOKEN                # 6 masked tokens, N = 6
    assert float(sum(totals)) == pytest.approx(want_total, rel=1e-6)
    assert len(totals) == (2 if packing else 1)
    # gradient w.r.t. the logprob of each masked token, by hand: d pg/d lp = -A r where the unclipped
    # branch is active (r = 1.1, 0.5, 1.0), 0 where the clipped branch wins (r = 1.5, 0.7, 1.3);
    # d kl/d lp = 1 - exp(k);  all divided by N.  Through log-softmax, d lp/d table[tok][v] = 1[v=label] - P[tok][v];
    # the entropy term contributes -coef/N * dH/dtable.  Checked on one table entry that only the
    # s0 position 1 token (tok 2 -> label 3, r = 1.1, A = 2) and s1 position 2 (unmasked) touch... tok 2 appears
    # at s0 pos 1 (masked) and s1 pos 2 (not masked), so row 2 of the table gets exactly one token's gradient.
    g_lp = (-2.0 * 1.1 + 0.05 * (1.0 - math.exp(-0.1))) / N_RESPONSE_TOKENS
    p_row = [2.0 ** -Q_EXP[(v - 2) % 7] for v in range(7)]
    # dH/dz_v = -p_v (log p_v + H)
    want_row = [g_lp * ((1.0 if v == 3 else 0.0) - p_row[v])
                - 0.01 / N_RESPONSE_TOKENS * (-p_row[v] * (math.log(p_row[v]) + ENTROPY)) for v in range(7)]
    assert model.table.grad[2].tolist() == pytest.approx(want_row, rel=1e-6, abs=1e-12)
    # tokens 0 (padding) and 5 (s0's last position, masked out by the zeroed last column) get no gradient
    assert model.table.grad[0].abs().max() == 0 and model.table.grad[5].abs().max() == 0


def test_train_step_entropy_off_means_no_entropy_gradient():
    model = ToyModel()
    stats, _ = opl.train_step(model, samples(True), packing=False, module_args={"entropy_coef": 0.0, "kl_coef": 0.0},
                              train_micro_batch_size=3)
    assert stats["entropy_loss"] == pytest.approx(ENTROPY, rel=1e-6)       # still reported (policy_trainer.py:226-228)
    g_lp = (-2.0 * 1.1) / N_RESPONSE_TOKENS
    p_row = [2.0 ** -Q_EXP[(v - 2) % 7] for v in range(7)]
    want_row = [g_lp * ((1.0 if v == 3 else 0.0) - p_row[v]) for v in range(7)]
    assert model.table.grad[2].tolist() == pytest.approx(want_row, rel=1e-6, abs=1e-12)


@pytest.mark.parametrize("packing", [False, True])
def test_train_step_sequence_level_policy(packing):
    """GSPO on the loop (loss_gallery.py:35-74): every token of a sequence carries the sequence's ratio
    exp(mean over its masked positions of lp - old); by hand from the RATIO table above
        s0: masked positions 1,2,3, ratios 1.1, 1.5, 0.5  -> rho0 = (1.1 * 1.5 * 0.5) ** (1/3) = 0.825 ** (1/3)
        s1: masked positions 0,1,   ratios 0.7, 1.0       -> rho1 = sqrt(0.7)
        s2: masked position 0,      ratio 1.3             -> rho2 = 1.3
    clip range [0.8, 1.2]:  s0 (A=+2) unclipped: -2 rho0 per token;  s1 (A=-1): rho1 inside: +rho1 per token;
    s2 (A=+0.5): max(-0.65, -0.6) = -0.6, clipped, no gradient.  d s_t / d lp_t = 1 (no 1/|y| factor), so the
    gradient w.r.t. a masked token's logprob of s0 is -2 rho0 / N."""
    rho0, rho1 = 0.825 ** (1.0 / 3.0), math.sqrt(0.7)
    pg = (3 * (-2.0 * rho0) + 2 * rho1 - 0.6) / N_RESPONSE_TOKENS
    model = ToyModel()
    kw = dict(max_token_in_seq=6) if packing else dict(train_micro_batch_size=3)
    args = {"entropy_coef": 0.0, "kl_coef": 0.05, "use_group_sequence_policy": True}
    stats, totals = opl.train_step(model, samples(True), packing=packing, module_args=args, **kw)
    assert stats["pg_loss"] == pytest.approx(pg, rel=1e-6)
    assert stats["kl_loss"] == pytest.approx(KL_TOKEN, rel=1e-6)
    assert float(sum(totals)) == pytest.approx(pg + 0.05 * KL_TOKEN, rel=1e-6)
    # table row 2 is touched by one masked token only (s0 position 1, label 3), as in the token-level test
    g_lp = (-2.0 * rho0 + 0.05 * (1.0 - math.exp(-0.1))) / N_RESPONSE_TOKENS
    p_row = [2.0 ** -Q_EXP[(v - 2) % 7] for v in range(7)]
    want_row = [g_lp * ((1.0 if v == 3 else 0.0) - p_row[v]) for v in range(7)]
    assert model.table.grad[2].tolist() == pytest.approx(want_row, rel=1e-6, abs=1e-12)
    # s2's only masked token (tok 3 -> label 4) is clipped: its row gets the KL gradient only ... tok 3 also sits at
    # s0 position 2 (masked, label 4, unclipped sequence), so row 3 holds s0's term plus s2's KL term
    g_s0 = (-2.0 * rho0 + 0.05 * (1.0 - math.exp(-0.1))) / N_RESPONSE_TOKENS
    g_s2 = (0.05 * (1.0 - math.exp(-0.1))) / N_RESPONSE_TOKENS
    p_row3 = [2.0 ** -Q_EXP[(v - 3) % 7] for v in range(7)]
    want_row3 = [(g_s0 + g_s2) * ((1.0 if v == 4 else 0.0) - p_row3[v]) for v in range(7)]
    assert model.table.grad[3].tolist() == pytest.approx(want_row3, rel=1e-6, abs=1e-12)


def test_vision_language_inputs_are_carried_through():
    """model_type = 'vlm' (policy_trainer.py:104-107,119-125,146-152; trainer_utils.py:76-92,176-187), by hand on
    two samples: s0 prompt 3 + response 2 with prompt position channels t = [0,1,2], h = [0,0,1], w = [0,1,0];
    s1 prompt 2 + response 1 with channels [0,1], [0,0], [0,1].  Each channel continues counting from its
    maximum + 1 over the rest of the padded row (S = 5):
        s0: t [0,1,2,3,4]  h [0,0,1,2,3]  w [0,1,0,2,3]
        s1: t [0,1,2,3,4]  h [0,0,1,2,3]  w [0,1,2,3,4]
    Padded batches keep the [3, B, S] tensor; packed ones unpad every channel with the same indices
    (s0's five positions, s1's three) into [3, 1, 8], and with transformers >= 4.55 the first channel is
    repeated in front ([4, 1, 8]).  pixel_values of the samples are concatenated, image_grid_thw too."""
    def vl_samples():
        out = []
        for toks, p, r, pos, n_patch in (([1, 2, 3, 4, 5], 3, 2, [[0, 1, 2], [0, 0, 1], [0, 1, 0]], 4),
                                         ([6, 1, 2], 2, 1, [[0, 1], [0, 0], [0, 1]], 2)):
            out.append({"all_tokens": torch.tensor(toks), "prompt_token_length": p, "response_token_length": r,
                        "position_ids": pos, "pixel_values": torch.full((n_patch, 3), float(len(toks))),
                        "image_grid_thw": torch.tensor([[1, 2, n_patch // 2]])})
        return out
    want_padded = [[[0, 1, 2, 3, 4], [0, 1, 2, 3, 4]], [[0, 0, 1, 2, 3], [0, 0, 1, 2, 3]], [[0, 1, 0, 2, 3], [0, 1, 2, 3, 4]]]
    _, mbs = opl.preprocess_data_list(vl_samples(), False, packing=False, generate_micro_batch_size=2, model_type="vlm")
    mb = mbs[0]
    assert mb["position_ids"].tolist() == want_padded
    assert mb["pixel_values"].shape == (6, 3) and mb["pixel_values"][:, 0].tolist() == [5.0] * 4 + [3.0] * 2
    assert mb["image_grid_thw"].tolist() == [[1, 2, 2], [1, 2, 1]]
    assert mb["all_tokens"].tolist() == [[1, 2, 3, 4, 5], [6, 1, 2, 0, 0]]
    want_packed = [[[0, 1, 2, 3, 4, 0, 1, 2]], [[0, 0, 1, 2, 3, 0, 0, 1]], [[0, 1, 0, 2, 3, 0, 1, 2]]]
    _, mbs = opl.preprocess_data_list(vl_samples(), False, packing=True, max_token_in_seq=9, model_type="vlm")
    assert len(mbs) == 1 and mbs[0]["position_ids"].tolist() == want_packed
    assert mbs[0]["all_tokens"].tolist() == [[1, 2, 3, 4, 5, 6, 1, 2]] and mbs[0]["labels"].tolist() == [[2, 3, 4, 5, 6, 1, 2, 1]]
    _, mbs = opl.preprocess_data_list(vl_samples(), False, packing=True, max_token_in_seq=9, model_type="vlm",
                                      prepend_text_position_channel=True)
    assert mbs[0]["position_ids"].tolist() == [want_packed[0]] + want_packed
    # the model is called with the image tensors (policy_trainer.py:206-214)
    seen = {}

    def model(ids, pos, pixel_values=None, image_grid_thw=None):
        seen.update(pos=tuple(pos.shape), pix=tuple(pixel_values.shape), grid=image_grid_thw.tolist())
        return ToyModel()(ids, pos)
    opl.forward_step(model, vl_samples(), packing=True, trainable=True, max_token_in_seq=9, model_type="vlm")
    assert seen == {"pos": (3, 1, 8), "pix": (6, 3), "grid": [[1, 2, 2], [1, 2, 1]]}
