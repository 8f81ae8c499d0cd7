"""The Hugging Face patch glue and the packing helpers.

CPU part: parameter names equal Hugging Face's (stock checkpoints load), in-place patching, mask
reduction, packing round trips, loud failure without a GPU.  GPU part: a two-layer model against
the golden last hidden state written by Hugging Face's eager model, the eager fallback for
``output_attentions``, and a bf16 encoder against Hugging Face eager run on the same device."""
import os

import numpy as np
import pytest
import torch

transformers = pytest.importorskip("transformers")
from transformers import DebertaV2Config  # noqa: E402
from transformers.models.deberta_v2.modeling_deberta_v2 import DebertaV2Model, DisentangledSelfAttention  # noqa: E402

from golden_inputs import fill_params, tiny_model_config, tiny_model_inputs  # noqa: E402
from turbodeberta_amd import padding  # noqa: E402
from turbodeberta_amd.model import (FlashDebertaV2Model, FlashDisentangledSelfAttention, patch_model)  # noqa: E402


def _tiny():
    return DebertaV2Config(**tiny_model_config())


def test_parameter_names_match_hugging_face():
    ours, theirs = FlashDebertaV2Model(_tiny()), DebertaV2Model(_tiny())
    assert list(ours.state_dict()) == list(theirs.state_dict())
    ours.load_state_dict(theirs.state_dict(), strict=True)
    assert sum(isinstance(m, FlashDisentangledSelfAttention) for m in ours.modules()) == 2


def test_patch_model_in_place():
    m = DebertaV2Model(_tiny())
    before = {k: v.clone() for k, v in m.state_dict().items()}
    assert patch_model(m) is m
    assert all(type(x) is not DisentangledSelfAttention for x in m.modules())
    assert sum(isinstance(x, FlashDisentangledSelfAttention) for x in m.modules()) == 2
    assert all(torch.equal(v, before[k]) for k, v in m.state_dict().items())


def test_task_heads_have_hugging_face_parameters():
    import transformers.models.deberta_v2.modeling_deberta_v2 as hf
    from turbodeberta_amd import model as ours
    cfg = DebertaV2Config(**dict(tiny_model_config(), num_labels=3))
    for name in ("ForMaskedLM", "ForSequenceClassification", "ForTokenClassification", "ForQuestionAnswering",
                 "ForMultipleChoice"):
        theirs = getattr(hf, "DebertaV2" + name)(cfg)
        mine = getattr(ours, "FlashDebertaV2" + name)(cfg)
        assert list(mine.state_dict()) == list(theirs.state_dict()), name
        mine.load_state_dict(theirs.state_dict(), strict=True)
        assert isinstance(mine.deberta, FlashDebertaV2Model) and isinstance(mine.deberta.encoder, ours.FlashDebertaV2Encoder)
        assert sum(isinstance(m, FlashDisentangledSelfAttention) for m in mine.modules()) == 2
        assert all(type(m) is not DisentangledSelfAttention for m in mine.modules())


def test_forward_without_gpu_fails_loudly():
    m = FlashDebertaV2Model(_tiny()).eval()
    ids, mask = tiny_model_inputs()
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        with torch.no_grad():
            m(input_ids=torch.from_numpy(ids), attention_mask=torch.from_numpy(mask))


def test_key_padding_mask_and_unpad_data():
    m2 = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1], [1, 0, 0, 0, 0]])
    ext = m2.unsqueeze(1).unsqueeze(2)
    m4 = ext * ext.squeeze(-2).unsqueeze(-1)                      # what the HF encoder builds
    for m in (m2, m4, m4[:, 0]):
        assert torch.equal(padding.key_padding_mask(m), m2)
        assert padding.sequence_lengths(m).tolist() == [3, 5, 1]
    idx, cu, mx = padding._get_unpad_data(m4)
    assert cu.dtype == torch.int32 and cu.tolist() == [0, 3, 8, 9] and mx == 5
    assert idx.tolist() == [0, 1, 2, 5, 6, 7, 8, 9, 10]


def test_pack_unpack_round_trip():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 5, 2, 4, generator=g)
    m2 = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1], [1, 0, 0, 0, 0]])
    packed, idx, cu, mx = padding.unpad_input(x, m2)
    assert packed.shape == (9, 2, 4) and torch.equal(packed[3:8], x[1])
    back = padding.pad_input(packed, idx, 3, 5)
    assert torch.equal(back, x * m2[:, :, None, None])
    q, k, v, pk, pq, idx2, (cq, ck), (mq, mk) = padding._upad_input(x, x, x, None, None, m2, 5, 2)
    assert torch.equal(q, packed) and pk is None and torch.equal(cq, cu) and mq == 5


def test_mask_shapes_accepted_and_rejected():
    from turbodeberta_amd.model import _mask_info
    m2 = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1], [1, 0, 0, 0, 0]])
    outer = m2[:, :, None] * m2[:, None, :]
    row = m2[:, None, None, :]                                    # the "extended" key mask [B, 1, 1, L]
    accepted = (m2, outer, outer[:, None], outer[:, None].expand(3, 4, 5, 5), row, row.expand(3, 4, 1, 5), m2[:, None, :])
    for m in accepted:
        info = _mask_info(m.clone())
        assert info.lengths.tolist() == [3, 5, 1] and info.total == 9, tuple(m.shape)
        assert torch.equal(padding.key_padding_mask(m), m2)
    # a broadcast key mask must not be read through a "diagonal" of its single row
    assert _mask_info(torch.ones(2, 1, 1, 7)).lengths.tolist() == [7, 7]
    # shapes with no token axis to read
    for bad in (torch.ones(3, 1, 2, 5), torch.ones(3, 4, 5), torch.ones(3, 5, 4)):
        with pytest.raises(ValueError, match="last two dimensions"):
            _mask_info(bad)
    # heads that differ: only head 0 would have been looked at
    per_head = outer[:, None].repeat(1, 2, 1, 1)
    per_head[1, 1, 4, 4] = 0
    with pytest.raises(ValueError, match="right padded"):
        _mask_info(per_head)
    per_head_row = row.repeat(1, 2, 1, 1)
    per_head_row[0, 1, 0, 2] = 0
    with pytest.raises(ValueError, match="right padded"):
        _mask_info(per_head_row)
    # holes, left padding, a square mask that is not an outer product
    for bad in (torch.tensor([[1, 0, 1, 0]]), torch.tensor([[0, 1, 1, 1]])):
        with pytest.raises(ValueError, match="right padded"):
            _mask_info(bad)
    causal = torch.tril(torch.ones(1, 4, 4, dtype=torch.long))
    with pytest.raises(ValueError, match="right padded"):
        _mask_info(causal)


def test_declared_masks_are_not_inspected():
    from turbodeberta_amd.model import _mask_info, declare_right_padded
    holes = torch.tensor([[1, 0, 1, 0], [1, 1, 1, 1]])                 # would be refused if it were looked at
    lengths = torch.tensor([2, 4], dtype=torch.int32)
    assert declare_right_padded(holes, lengths) is holes
    info = _mask_info(holes)
    assert info.lengths is lengths and info.total is None
    assert _mask_info(declare_right_padded(holes, lengths, total=6)).total == 6
    holes[1, 1] = 0                                                    # an in-place edit voids the declaration
    with pytest.raises(ValueError, match="right padded"):
        _mask_info(holes)
    for bad in (lengths.long(), lengths[:1], lengths[None]):
        with pytest.raises(ValueError, match="lengths"):
            declare_right_padded(holes, bad)


def test_model_passes_the_hidden_state_wish_as_an_argument():
    """The model tells the encoder per call (not through module state) whether the layers' outputs are wanted."""
    m = FlashDebertaV2Model(_tiny()).eval()
    seen = []

    class Stop(Exception):
        pass

    def spy(hidden_states, attention_mask, **kw):
        seen.append(kw.get("intermediate_states", True))
        raise Stop

    m.encoder.forward = spy
    ids, mask = (torch.from_numpy(a) for a in tiny_model_inputs())
    for wish, expected in ((None, False), (False, False), (True, True)):
        with pytest.raises(Stop):
            m(input_ids=ids, attention_mask=mask, output_hidden_states=wish)
        assert seen[-1] is expected
    assert not any(k.startswith("_tdb_all") for k in vars(m.encoder))
    with pytest.raises(ValueError, match="exactly one"):
        m(input_ids=ids, inputs_embeds=torch.zeros(2, 3, 4))


# ------------------------------------------------------------------------------------- GPU

@pytest.mark.gpu
def test_tiny_model_matches_hf_golden(golden_dir):
    cfg = _tiny()
    model = FlashDebertaV2Model(cfg).eval()
    fill_params(model)
    model = model.to("cuda:0")
    ids, mask = tiny_model_inputs()
    gold = torch.from_numpy(np.load(os.path.join(golden_dir, "hf_tiny_model.npz"))["last_hidden_state"])
    print("[case] tiny model fp32", flush=True)
    with torch.no_grad():
        out = model(input_ids=torch.from_numpy(ids).cuda(), attention_mask=torch.from_numpy(mask).cuda()).last_hidden_state
    out = out.float().cpu()
    valid = torch.from_numpy(mask).bool()
    rel = (out[valid] - gold[valid]).abs().max() / gold[valid].abs().max()
    assert rel <= 1e-4, rel


@pytest.mark.gpu
def test_declared_mask_gives_the_same_result_without_packing():
    """A mask declared right padded (no inspection, no host synchronisation) without a token count keeps the padded
    layout; with the count the encoder packs.  Both must reproduce the inspected-mask result on the valid tokens."""
    from turbodeberta_amd.model import declare_right_padded
    model = FlashDebertaV2Model(_tiny()).eval()
    fill_params(model)
    model = model.to("cuda:0")
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    valid = mask.bool()
    lengths = mask.sum(-1, dtype=torch.int32)
    with torch.no_grad():
        want = model(input_ids=ids, attention_mask=mask.clone()).last_hidden_state
        print("[case] declared mask, padded layout", flush=True)
        padded = model(input_ids=ids, attention_mask=declare_right_padded(mask.clone(), lengths)).last_hidden_state
        print("[case] declared mask, packed layout", flush=True)
        packed = model(input_ids=ids, attention_mask=declare_right_padded(mask.clone(), lengths, int(lengths.sum()))
                       ).last_hidden_state
    assert torch.equal(packed[valid], want[valid])
    assert torch.allclose(padded[valid], want[valid], atol=2e-5, rtol=0)


@pytest.mark.gpu
def test_output_attentions_falls_back_to_eager():
    cfg = _tiny()
    ours, theirs = FlashDebertaV2Model(cfg).eval(), DebertaV2Model(cfg).eval()
    fill_params(ours)
    theirs.load_state_dict(ours.state_dict())
    ours, theirs = ours.cuda(), theirs.cuda()
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask, output_attentions=True)
        b = theirs(input_ids=ids, attention_mask=mask, output_attentions=True)
    assert len(a.attentions) == 2 and torch.allclose(a.attentions[0], b.attentions[0], atol=1e-5)
    assert torch.allclose(a.last_hidden_state, b.last_hidden_state, atol=1e-4)


@pytest.mark.gpu
def test_bf16_encoder_matches_hf_eager_on_device():
    # v3-base-like widths, 3 layers: patched model vs the unpatched Hugging Face model, both bf16 on the GPU
    cfg = DebertaV2Config(vocab_size=1000, hidden_size=768, num_hidden_layers=3, num_attention_heads=12,
                          intermediate_size=3072, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                          max_position_embeddings=512, type_vocab_size=0, relative_attention=True, position_buckets=256,
                          max_relative_positions=512, share_att_key=True, pos_att_type=["c2p", "p2c"],
                          norm_rel_ebd="layer_norm", position_biased_input=False, layer_norm_eps=1e-7)
    torch.manual_seed(0)
    truth = DebertaV2Model(cfg).eval()
    fill_params(truth, seed=5)
    theirs = DebertaV2Model(cfg).eval()
    theirs.load_state_dict(truth.state_dict())
    ours = patch_model(DebertaV2Model(cfg).eval())
    ours.load_state_dict(truth.state_dict())
    truth = truth.to("cuda:0")                                            # float32 eager: the yardstick
    theirs, ours = theirs.to("cuda:0", torch.bfloat16), ours.to("cuda:0", torch.bfloat16)
    rs = np.random.RandomState(1)
    lens = np.array([300, 128, 77, 299])
    ids = torch.from_numpy(rs.randint(1, 1000, size=(4, 300))).cuda()
    mask = torch.from_numpy((np.arange(300)[None] < lens[:, None]).astype(np.int64)).cuda()
    print("[case] bf16 3-layer encoder", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask).last_hidden_state.float()
        b = theirs(input_ids=ids, attention_mask=mask).last_hidden_state.float()
        t = truth(input_ids=ids, attention_mask=mask).last_hidden_state
    valid = mask.bool()
    # Hidden states are LayerNorm outputs of order 1, so one bf16 ulp is 8e-3.  The patched model must be as close
    # to the float32 model as Hugging Face's own bf16 eager run is (it keeps fp32 scores, so it is usually closer).
    err_ours = (a[valid] - t[valid]).abs()
    err_hf = (b[valid] - t[valid]).abs()
    assert err_ours.mean().item() <= 1.25 * err_hf.mean().item() + 1e-4, (err_ours.mean().item(), err_hf.mean().item())
    assert err_ours.max().item() <= 1.5 * err_hf.max().item() + 1e-3, (err_ours.max().item(), err_hf.max().item())
    assert (a[valid] - b[valid]).abs().max().item() <= 1e-1


@pytest.mark.gpu
def test_eval_caches_follow_weight_updates():
    """Eval-mode caches (position tables, fused Q/K/V weight, lengths): the cached forward equals the uncached one
    (grad mode on takes the per-call path), a repeated call hits the caches and gives the same bits, and an in-place
    weight update or a new mask invalidates them."""
    cfg = _tiny()
    model = FlashDebertaV2Model(cfg).eval()
    fill_params(model)
    model = model.to("cuda:0")
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    att = model.encoder.layer[0].attention.self
    print("[case] eval caches", flush=True)
    uncached = model(input_ids=ids, attention_mask=mask).last_hidden_state.detach()     # grad mode on: no caches
    assert "_tdb_tables" not in att.__dict__ and "_tdb_qkv" not in att.__dict__
    with torch.no_grad():
        first = model(input_ids=ids, attention_mask=mask).last_hidden_state
        assert "_tdb_tables" in att.__dict__ and "_tdb_qkv" in att.__dict__
        tables = att.__dict__["_tdb_tables"][1][0]
        second = model(input_ids=ids, attention_mask=mask).last_hidden_state
        assert att.__dict__["_tdb_tables"][1][0] is tables                               # cache hit
    valid = mask.bool()
    assert torch.equal(first, second)
    assert (first[valid] - uncached[valid]).abs().max() <= 1e-5 * uncached[valid].abs().max()
    with torch.no_grad():
        att.key_proj.weight.mul_(1.5)                                                    # bumps the version counter
        changed = model(input_ids=ids, attention_mask=mask).last_hidden_state
        assert att.__dict__["_tdb_tables"][1][0] is not tables
    fresh = model(input_ids=ids, attention_mask=mask).last_hidden_state.detach()
    assert (changed[valid] - fresh[valid]).abs().max() <= 1e-5 * fresh[valid].abs().max()
    assert (changed[valid] - first[valid]).abs().max() > 1e-3
    with torch.no_grad():                                                                # relative embeddings updated in place
        model.encoder.rel_embeddings.weight[:, :16].mul_(-3.0)                           # (not a rescaling: the LayerNorm would undo one)
        moved = model(input_ids=ids, attention_mask=mask).last_hidden_state
    fresh2 = model(input_ids=ids, attention_mask=mask).last_hidden_state.detach()
    assert (moved[valid] - fresh2[valid]).abs().max().item() <= 1e-5 * fresh2[valid].abs().max().item()
    assert (moved[valid] - changed[valid]).abs().max().item() > 1e-4
    with torch.no_grad():                                                                # shorter sequences, new mask
        mask2 = mask.clone()
        mask2[:, -3:] = 0
        a = model(input_ids=ids, attention_mask=mask2).last_hidden_state
    b = model(input_ids=ids, attention_mask=mask2).last_hidden_state.detach()
    v2 = mask2.bool()
    assert (a[v2] - b[v2]).abs().max() <= 1e-5 * b[v2].abs().max()


@pytest.mark.gpu
@pytest.mark.parametrize("conv", [0, 3])
def test_packed_encoder_matches_hf_eager_and_padded_path(conv):
    """Eval mode keeps a batch with padding packed through the whole encoder.  fp32, 3 layers (with and without the
    convolution after the first layer): against Hugging Face's eager model on the same device, against the padded
    path of the same model, every layer's output when asked for, zeros at padded positions, and an unpadded batch."""
    cfg = DebertaV2Config(**dict(tiny_model_config(), num_hidden_layers=3, conv_kernel_size=conv, conv_act="gelu"))
    theirs = DebertaV2Model(cfg).eval()
    fill_params(theirs, seed=11)
    ours = FlashDebertaV2Model(cfg).eval()
    ours.load_state_dict(theirs.state_dict())
    ours, theirs = ours.to("cuda:0"), theirs.to("cuda:0")
    rs = np.random.RandomState(3)
    B, L = 5, 40
    lens = np.array([40, 1, 17, 33, 8])
    ids = torch.from_numpy(rs.randint(1, cfg.vocab_size, size=(B, L))).cuda()
    mask = torch.from_numpy((np.arange(L)[None] < lens[:, None]).astype(np.int64)).cuda()
    valid = mask.bool()
    print(f"[case] packed encoder conv={conv}", flush=True)
    with torch.no_grad():
        want = theirs(input_ids=ids, attention_mask=mask, output_hidden_states=True)
        got = ours(input_ids=ids, attention_mask=mask, output_hidden_states=True)
        ours.encoder.pack_sequences = False
        padded = ours(input_ids=ids, attention_mask=mask, output_hidden_states=True)
        ours.encoder.pack_sequences = True
        last_only = ours(input_ids=ids, attention_mask=mask)
    assert len(got.hidden_states) == len(want.hidden_states) == 4
    for g, p, w in zip(got.hidden_states, padded.hidden_states, want.hidden_states):
        scale = w[valid].abs().max().item()
        assert (g[valid] - w[valid]).abs().max().item() <= 1e-4 * scale
        assert (g[valid] - p[valid]).abs().max().item() <= 1e-5 * scale
    assert bool(torch.equal(got.last_hidden_state, got.hidden_states[-1]))
    assert got.last_hidden_state[~valid].abs().max().item() == 0.0
    assert last_only.hidden_states is None
    # (the library convolution may pick another algorithm on a later call: equal to rounding, not to the bit)
    assert (last_only.last_hidden_state - got.last_hidden_state).abs().max().item() <= 1e-5 * scale
    # a batch without padding takes the padded path (nothing to pack) and still agrees
    full = torch.ones_like(mask)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=full).last_hidden_state
        b = theirs(input_ids=ids, attention_mask=full).last_hidden_state
    assert (a - b).abs().max().item() <= 1e-4 * b.abs().max().item()


@pytest.mark.gpu
def test_sequence_classifier_matches_hf_eager():
    from transformers.models.deberta_v2.modeling_deberta_v2 import DebertaV2ForSequenceClassification
    from turbodeberta_amd.model import FlashDebertaV2ForSequenceClassification
    cfg = DebertaV2Config(**dict(tiny_model_config(), num_labels=4))
    theirs = DebertaV2ForSequenceClassification(cfg).eval()
    fill_params(theirs, seed=8)
    ours = FlashDebertaV2ForSequenceClassification(cfg).eval()
    ours.load_state_dict(theirs.state_dict())
    ours, theirs = ours.to("cuda:0"), theirs.to("cuda:0")
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    print("[case] sequence classifier", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask).logits
        b = theirs(input_ids=ids, attention_mask=mask).logits
    assert a.shape == b.shape == (ids.shape[0], 4)
    assert (a - b).abs().max().item() <= 1e-4 * b.abs().max().item()


@pytest.mark.gpu
def test_patch_model_packs_a_task_head():
    """``patch_model`` on a Hugging Face task model: the encoder inside runs packed, logits equal eager's."""
    from transformers.models.deberta_v2.modeling_deberta_v2 import DebertaV2ForTokenClassification
    from turbodeberta_amd.model import FlashDebertaV2Encoder
    cfg = DebertaV2Config(**dict(tiny_model_config(), num_labels=5))
    theirs = DebertaV2ForTokenClassification(cfg).eval()
    fill_params(theirs, seed=2)
    ours = DebertaV2ForTokenClassification(cfg).eval()
    ours.load_state_dict(theirs.state_dict())
    assert isinstance(patch_model(ours).deberta.encoder, FlashDebertaV2Encoder)
    ours, theirs = ours.to("cuda:0"), theirs.to("cuda:0")
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    print("[case] patched token classifier", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask).logits
        b = theirs(input_ids=ids, attention_mask=mask).logits
    valid = mask.bool()
    assert (a[valid] - b[valid]).abs().max().item() <= 1e-4 * b[valid].abs().max().item()


@pytest.mark.gpu
def test_query_states_from_another_tensor():
    """The enhanced-mask-decoder call shape (modeling_deberta_v2.py:772-788): queries projected from ``query_states``,
    keys and values from ``hidden_states``, against the eager module on the device (fp32)."""
    cfg = _tiny()
    theirs = DisentangledSelfAttention(cfg).eval()
    fill_params(theirs, seed=21)
    ours = FlashDisentangledSelfAttention(cfg).eval()
    ours.load_state_dict(theirs.state_dict())
    ours, theirs = ours.to("cuda:0"), theirs.to("cuda:0")
    g = torch.Generator().manual_seed(4)
    B, L = 3, 24
    hidden = torch.randn(B, L, cfg.hidden_size, generator=g).cuda()
    queries = torch.randn(B, L, cfg.hidden_size, generator=g).cuda()
    rel = torch.randn(2 * cfg.position_buckets, cfg.hidden_size, generator=g).cuda()
    lens = torch.tensor([24, 9, 17])
    mask2 = (torch.arange(L)[None] < lens[:, None]).long().cuda()
    ext = mask2.unsqueeze(1).unsqueeze(2)
    mask4 = ext * ext.squeeze(-2).unsqueeze(-1)
    print("[case] query_states", flush=True)
    with torch.no_grad():
        want = theirs(hidden, mask4, False, query_states=queries, rel_embeddings=rel)[0]
        got = ours(hidden, mask4, False, query_states=queries, rel_embeddings=rel)[0]
    valid = mask2.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 1e-4 * want[valid].abs().max().item()


def _pair(cls_name, cfg, seed, flash_name=None):
    """(ours, theirs) on the GPU, fp32, eval: the Hugging Face class and the fused class of the same name with the
    same seeded parameters."""
    import transformers.models.deberta_v2.modeling_deberta_v2 as hf
    from turbodeberta_amd import model as fused
    theirs = getattr(hf, "DebertaV2" + cls_name)(cfg).eval()
    fill_params(theirs, seed=seed)
    ours = getattr(fused, flash_name or ("FlashDebertaV2" + cls_name))(cfg).eval()
    ours.load_state_dict(theirs.state_dict())
    return ours.to("cuda:0"), theirs.to("cuda:0")


@pytest.mark.gpu
def test_masked_lm_matches_hf_eager():
    """FlashDebertaV2ForMaskedLM (reference model.py:244-262): logits over the vocabulary on valid tokens."""
    cfg = _tiny()
    ours, theirs = _pair("ForMaskedLM", cfg, seed=31)
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    print("[case] masked LM head", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask).logits
        b = theirs(input_ids=ids, attention_mask=mask).logits
    valid = mask.bool()
    assert a.shape == b.shape == (*ids.shape, cfg.vocab_size)
    assert (a[valid] - b[valid]).abs().max().item() <= 1e-4 * b[valid].abs().max().item()


@pytest.mark.gpu
def test_question_answering_matches_hf_eager():
    """FlashDebertaV2ForQuestionAnswering (reference model.py:290-301): start / end logits on valid tokens."""
    cfg = DebertaV2Config(**dict(tiny_model_config(), num_labels=2))
    ours, theirs = _pair("ForQuestionAnswering", cfg, seed=32)
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    print("[case] question answering head", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask)
        b = theirs(input_ids=ids, attention_mask=mask)
    valid = mask.bool()
    for x, y in ((a.start_logits, b.start_logits), (a.end_logits, b.end_logits)):
        assert x.shape == y.shape == tuple(ids.shape)
        assert (x[valid] - y[valid]).abs().max().item() <= 1e-4 * y[valid].abs().max().item()


@pytest.mark.gpu
def test_multiple_choice_matches_hf_eager():
    """FlashDebertaV2ForMultipleChoice (reference model.py:303-314): ids [batch, choices, L]; one logit per choice."""
    cfg = _tiny()
    ours, theirs = _pair("ForMultipleChoice", cfg, seed=33)
    rs = np.random.RandomState(5)
    B, C, L = 2, 3, 24
    lens = rs.randint(1, L + 1, size=(B, C))
    mask = torch.from_numpy((np.arange(L)[None, None] < lens[:, :, None]).astype(np.int64)).cuda()
    ids = torch.from_numpy(rs.randint(1, cfg.vocab_size, size=(B, C, L))).cuda() * mask
    print("[case] multiple choice head", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask).logits
        b = theirs(input_ids=ids, attention_mask=mask).logits
    assert a.shape == b.shape == (B, C)
    assert (a - b).abs().max().item() <= 1e-4 * b.abs().max().item()


@pytest.mark.gpu
def test_enhanced_mask_decoder_step():
    """The body of the ``z_steps > 1`` loop (modeling_deberta_v2.py:772-788): the last layer run again with the previous
    output as ``query_states``, the encoder's 4-D mask, its relative-position matrix and relative embeddings.  (The loop
    itself cannot run in transformers 5.15 -- it appends to a tuple -- for the eager model either, which this test
    records; the layer call it makes is compared directly.)"""
    cfg = _tiny()
    ours, theirs = _pair("Model", cfg, seed=34)
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    print("[case] enhanced mask decoder step", flush=True)
    with torch.no_grad():
        enc = theirs(input_ids=ids, attention_mask=mask, output_hidden_states=True)
        hidden, queries = enc.hidden_states[-2], enc.hidden_states[-1]
        rel = theirs.encoder.get_rel_embedding()
        mask4 = theirs.encoder.get_attention_mask(mask)
        rel_pos = theirs.encoder.get_rel_pos(hidden)
        want = theirs.encoder.layer[-1](hidden, mask4, output_attentions=False, query_states=queries,
                                        relative_pos=rel_pos, rel_embeddings=rel)[0]
        got = ours.encoder.layer[-1](hidden, mask4, output_attentions=False, query_states=queries,
                                     relative_pos=rel_pos, rel_embeddings=ours.encoder.get_rel_embedding())[0]
        theirs.z_steps = 2
        with pytest.raises(AttributeError):                                   # Hugging Face's own loop is dead code
            theirs(input_ids=ids, attention_mask=mask)
    valid = mask.bool()
    assert (got[valid] - want[valid]).abs().max().item() <= 1e-4 * want[valid].abs().max().item()
    assert (want[valid] - queries[valid]).abs().max().item() > 1e-3          # the step does something


@pytest.mark.gpu
@pytest.mark.parametrize("buckets", [-1, 0])
def test_model_without_log_buckets(buckets):
    """``position_buckets <= 0``: plain clamped relative positions, span = max_relative_positions
    (modeling_deberta_v2.py:170-176, :585-588)."""
    cfg = DebertaV2Config(**dict(tiny_model_config(), position_buckets=buckets, max_relative_positions=24))
    ours, theirs = _pair("Model", cfg, seed=35)
    ids, mask = tiny_model_inputs()                                             # L = 40 > max_relative_positions
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    print(f"[case] model with position_buckets={buckets}", flush=True)
    with torch.no_grad():
        a = ours(input_ids=ids, attention_mask=mask).last_hidden_state
        b = theirs(input_ids=ids, attention_mask=mask).last_hidden_state
    valid = mask.bool()
    assert (a[valid] - b[valid]).abs().max().item() <= 1e-4 * b[valid].abs().max().item()


@pytest.mark.gpu
def test_inference_mode_padded_and_unpadded():
    """Under ``torch.inference_mode()`` masks are inference tensors without a modification counter; both the packed
    path (batch with padding) and the padded path (batch without) must run and agree with ``no_grad``."""
    cfg = _tiny()
    ours, theirs = _pair("Model", cfg, seed=36)
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    full = torch.ones_like(mask)
    print("[case] inference mode", flush=True)
    with torch.no_grad():
        want_pad = theirs(input_ids=ids, attention_mask=mask).last_hidden_state
        want_full = theirs(input_ids=ids, attention_mask=full).last_hidden_state
    with torch.inference_mode():
        got_pad = ours(input_ids=ids, attention_mask=mask).last_hidden_state
        got_full = ours(input_ids=ids, attention_mask=full).last_hidden_state
        again = ours(input_ids=ids.clone(), attention_mask=mask.clone()).last_hidden_state   # masks created inside
    valid = mask.bool()
    assert (got_pad[valid] - want_pad[valid]).abs().max().item() <= 1e-4 * want_pad[valid].abs().max().item()
    assert (got_full - want_full).abs().max().item() <= 1e-4 * want_full.abs().max().item()
    assert torch.equal(again, got_pad)


@pytest.mark.gpu
def test_masks_that_are_not_right_padded_raise():
    """Left padding, holes and a 4-D mask that is not ``m_i * m_j`` cannot be expressed as per-sequence lengths: the
    fused paths refuse them instead of attending to the wrong tokens (eager Hugging Face handles them)."""
    cfg = _tiny()
    ours, _ = _pair("Model", cfg, seed=37)
    ids, mask = tiny_model_inputs()
    ids, mask = torch.from_numpy(ids).cuda(), torch.from_numpy(mask).cuda()
    left = torch.flip(mask, dims=[1])
    holes = mask.clone()
    holes[0, 5] = 0
    for bad in (left, holes):
        for pack in (True, False):
            ours.encoder.pack_sequences = pack
            with torch.no_grad(), pytest.raises(ValueError, match="right padded"):
                ours(input_ids=ids, attention_mask=bad)
    ours.encoder.pack_sequences = True
    att = ours.encoder.layer[0].attention.self
    hidden = torch.randn(3, 40, cfg.hidden_size, device="cuda:0")
    rel = ours.encoder.get_rel_embedding()
    ext = mask.unsqueeze(1).unsqueeze(2)
    m4 = (ext * ext.squeeze(-2).unsqueeze(-1)).clone()
    m4[0, 0, 3, 7] = 0                                                          # a real [L, L] pattern
    with torch.no_grad(), pytest.raises(ValueError, match="right padded"):
        att(hidden, m4, False, rel_embeddings=rel)


@pytest.mark.gpu
def test_config4_v3_large_encoder_b16_l512():
    """BASELINE config 4 at its stated shape: 24 layers x 1024, 16 heads x 64, FFN 4096, vocabulary 128100, buckets 256,
    max_rel 512, random N(0, 0.02) weights, bf16; ids [16, 512] with valid lengths uniform in [64, 512].  The patched
    model (reference model.py:204-242), packed and padded, must be as close to the float32 Hugging Face model on the
    same device as Hugging Face's own bf16 eager run is."""
    cfg = DebertaV2Config(vocab_size=128100, hidden_size=1024, num_hidden_layers=24, num_attention_heads=16,
                          intermediate_size=4096, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                          max_position_embeddings=512, type_vocab_size=0, relative_attention=True, position_buckets=256,
                          max_relative_positions=512, share_att_key=True, pos_att_type=["c2p", "p2c"],
                          norm_rel_ebd="layer_norm", position_biased_input=False, layer_norm_eps=1e-7,
                          initializer_range=0.02)
    torch.manual_seed(0)
    with torch.device("cuda:0"):
        truth = DebertaV2Model(cfg).eval()                                    # float32 eager: the yardstick
    import copy
    theirs = copy.deepcopy(truth).to(torch.bfloat16)
    ours = patch_model(copy.deepcopy(truth).to(torch.bfloat16))
    rs = np.random.RandomState(0)
    lens = rs.randint(64, 513, size=16)
    ids = torch.from_numpy(rs.randint(0, 128000, size=(16, 512))).cuda()
    mask = torch.from_numpy((np.arange(512)[None] < lens[:, None]).astype(np.int64)).cuda()
    valid = mask.bool()
    print("[case] config 4: v3-large-shaped encoder, b16 x L512, bf16", flush=True)
    with torch.no_grad():
        t = truth(input_ids=ids, attention_mask=mask).last_hidden_state
        b = theirs(input_ids=ids, attention_mask=mask).last_hidden_state.float()
        packed = ours(input_ids=ids, attention_mask=mask).last_hidden_state.float()
        ours.encoder.pack_sequences = False
        padded = ours(input_ids=ids, attention_mask=mask).last_hidden_state.float()
    assert packed[~valid].abs().max().item() == 0.0
    err_hf = (b[valid] - t[valid]).abs()
    for name, a in (("packed", packed), ("padded", padded)):
        assert torch.isfinite(a).all(), name
        err = (a[valid] - t[valid]).abs()
        print(f"  {name}: mean |err| {err.mean().item():.4e} (HF bf16 eager {err_hf.mean().item():.4e}), "
              f"max {err.max().item():.4e} (HF {err_hf.max().item():.4e})", flush=True)
        assert err.mean().item() <= 1.25 * err_hf.mean().item() + 1e-4, name
        assert err.max().item() <= 1.5 * err_hf.max().item() + 1e-3, name
    assert (packed[valid] - padded[valid]).abs().max().item() <= 1.5 * err_hf.max().item() + 1e-3
