"""The reference's optimizer-construction smoke test (unitest/test_optimizer_init.py:45-60: FP16Adam over a BERT built
from a local config) restated against this engine, extended by a few training iterations."""
import pytest
import torch

import patrickstar_amd as ps

pytestmark = pytest.mark.gpu


def test_engine_trains_a_small_bert():
    transformers = pytest.importorskip("transformers")
    cfg = transformers.BertConfig(
        vocab_size=512, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, intermediate_size=128,
        max_position_embeddings=64, num_labels=2, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
    )
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "Adam", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-6, "weight_decay": 0, "use_hybrid_adam": True}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 10, "loss_scale_window": 1000, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 32 * 1024,
        "release_after_init": False,
        "use_cpu_embedding": False,
    }
    engine, optimizer = ps.initialize_engine(
        model_func=lambda: transformers.BertForSequenceClassification(cfg), local_rank=0, config=config
    )
    client = engine.client
    n_params = sum(p.numel() for p in engine.module.parameters())
    pos = client.positions()
    assert len(pos) >= 3 and all(q.exp_avg is not None and q.exp_avg_sq is not None for q in pos)
    assert sum(client.chunk_tensor_index.used_numel(q.fp16) for q in pos) == n_params
    idx = client.chunk_tensor_index
    for p in engine.module.parameters():
        assert p.dtype == torch.half and p.is_cuda
        info = idx.get_tensor_info(p.ps_attr.data_id())
        for key in ("exp_avg", "exp_avg_sq"):
            sp = dict.__getitem__(optimizer.state[p], key)
            assert idx.get_tensor_info(sp.ps_attr.data_id()).start_offset == info.start_offset
        assert p.data_ptr() == client.chunk_list[info.chunk_id].payload.data_ptr() + 2 * info.start_offset

    ids = torch.randint(0, 512, (8, 32), device="cuda")
    labels = torch.randint(0, 2, (8,), device="cuda")
    losses = []
    for it in range(12):
        out = engine(input_ids=ids, labels=labels)
        loss = out.loss
        engine.backward(loss)
        optimizer.step()
        losses.append(float(loss.detach()))
    assert all(l == l for l in losses)  # finite
    assert losses[-1] < losses[0] * 0.8, losses  # it learns the 8 fixed examples
    steps = optimizer.state[next(engine.module.parameters())]["step"]
    assert steps + optimizer.loss_scaler.skipped_steps == 12
    sd = optimizer.state_dict()
    assert len(sd["state"]) == len(list(engine.module.parameters())) and "loss_scaler" in sd


def test_bert_base_at_the_reference_chunk_size_matches_the_oracle():
    """The model of the reference's construction test (unitest/test_optimizer_init.py:47-60: BertConfig() defaults with a
    small vocabulary, chunk size 32 Mi elements), trained for three iterations through the engine.  After every backward
    the fp16 chunk payloads hold the gradients; the oracle is stepped on exactly those and every payload must come out
    bit for bit the same (about 86 M parameters in 3 chunk positions)."""
    transformers = pytest.importorskip("transformers")
    import numpy as np

    import oracle
    from _harness import assert_bits_equal, tensor_spans

    cfg = transformers.BertConfig(vocab_size=10, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, num_labels=2)
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-4, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.01}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 12, "loss_scale_window": 1000, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 32 * 1024 * 1024,
    }
    engine, optimizer = ps.initialize_engine(
        model_func=lambda: transformers.BertForSequenceClassification(cfg), local_rank=0, config=config
    )
    client = engine.client
    cl = client.chunk_list
    pos = client.positions()
    n_params = sum(p.numel() for p in engine.module.parameters())
    assert n_params > 80e6 and len(pos) >= 3

    def snap(t):
        return t.detach().to("cpu", copy=True).numpy()

    mirror = [{"p32": snap(cl[q.fp32].payload), "m": snap(cl[q.exp_avg].payload), "v": snap(cl[q.exp_avg_sq].payload),
               "p16": snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    # one operator call per parameter tensor, in parameters() order, as the reference's loop makes them
    spans = tensor_spans(client, optimizer)
    assert len(spans) == len(list(engine.module.parameters())) > 190
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                                      tensors=spans)
    ids = torch.randint(0, 10, (4, 64), device="cuda")
    labels = torch.randint(0, 2, (4,), device="cuda")
    for it in range(3):
        loss = engine(input_ids=ids, labels=labels).loss
        engine.backward(loss)
        for q, c in zip(pos, mirror):
            c["p16"][...] = snap(cl[q.fp16].payload)
        optimizer.step()
        oopt.check_overflow()
        oopt.step()
        for i, (q, c) in enumerate(zip(pos, mirror)):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(snap(cl[cid].payload), c[key], f"iteration {it} position {i} {key}")
        assert optimizer.loss_scaler.loss_scale == oscaler.loss_scale
    assert np.isfinite(float(loss.detach()))


@pytest.mark.parametrize("use_cpu_embedding", [False, True])
def test_checkpoint_reload_reproduces_the_losses_exactly(use_cpu_embedding):
    """The reference's checkpoint test (unitest/test_checkpoint.py:95-181) on a small BERT: train 5 steps, save model and
    optimizer, train 5 more on recorded batches, reload, and require (a) the loss right after reloading to EQUAL the
    loss at the save point and (b) the loss after re-training on the same 5 batches to EQUAL the loss of the first
    run.  Both need the fp32 masters, m, v, the step counter and the loss-scaler state to come back bit for bit.
    The reference's test sets "use_cpu_embedding": True (:100): the three embedding tables are then fp32 parameters
    of PyTorch's own, updated from fp32 gradients and saved with the model as they are."""
    transformers = pytest.importorskip("transformers")
    cfg = transformers.BertConfig(
        vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, intermediate_size=128,
        max_position_embeddings=64, num_labels=2, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
    )
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "Adam", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-6, "weight_decay": 0, "use_hybrid_adam": True}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 10, "loss_scale_window": 4, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 32 * 1024,
        "use_cpu_embedding": use_cpu_embedding,
    }
    model, optimizer = ps.initialize_engine(
        model_func=lambda: transformers.BertForSequenceClassification(cfg), local_rank=0, config=config
    )
    emb = model.module.bert.embeddings
    assert emb.word_embeddings.weight.dtype == (torch.float if use_cpu_embedding else torch.half)
    assert (optimizer._make_plan()["kind"] == "each") == use_cpu_embedding
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)

    def batch():
        return (torch.randint(0, 256, (4, 32), device="cuda", generator=gen), torch.randint(0, 2, (4,), device="cuda", generator=gen))

    def train_one_step(b):
        loss = model(input_ids=b[0], labels=b[1])[0]
        model.backward(loss)
        optimizer.step()

    def evaluate(b):
        model.eval()
        with torch.no_grad():
            out = model(input_ids=b[0], labels=b[1])[0].item()
        model.train()
        return out

    batch0 = batch()
    for _ in range(5):
        train_one_step(batch())
    loss0 = evaluate(batch0)
    model_sd = model.state_dict()
    opt_sd = optimizer.state_dict()
    assert all(v.dtype == torch.float for k, v in model_sd.items() if "weight" in k or "bias" in k)  # the masters
    later = [batch() for _ in range(5)]
    for b in later:
        train_one_step(b)
    loss1 = evaluate(batch0)
    assert loss1 != loss0
    model.load_state_dict(model_sd)
    optimizer.load_state_dict(opt_sd)
    loss2 = evaluate(batch0)
    assert loss0 == loss2, f"Model checkpoint error. {loss0} vs {loss2}"
    for b in later:
        train_one_step(b)
    loss3 = evaluate(batch0)
    assert loss1 == loss3, f"Optimizer checkpoint error. {loss1} vs {loss3}"
    with pytest.raises(RuntimeError, match="strictly"):
        model.load_state_dict({"no.such.key": torch.zeros(1)}, strict=True)


def test_a_fine_tuning_schedule_that_thaws_layers_matches_the_oracle():
    """Only the classifier head and the last encoder layer train at first; the first encoder layer joins after three
    steps and the embeddings after five.  The reference counts state[p]["step"] per parameter
    (fp16_cpu_adam.py:571-574), so from then on every operator call carries its own tensor's step number: the head's
    stand at 4, 5, 6 ..., layer 0's at 1, 2, 3 ..., the embeddings' at 1, 2.  Dynamic loss scale with a skipped step in
    the middle; bit for bit against the oracle, which is told the same schedule."""
    transformers = pytest.importorskip("transformers")
    import oracle
    from _harness import assert_bits_equal, tensor_spans

    cfg = transformers.BertConfig(
        vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, intermediate_size=128,
        max_position_embeddings=64, num_labels=2, hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
    )
    torch.manual_seed(0)
    config = {
        "optimizer": {"type": "AdamW", "params": {"lr": 1e-3, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.01}},
        "fp16": {"enabled": True, "loss_scale": 0, "initial_scale_power": 10, "loss_scale_window": 4, "hysteresis": 2, "min_loss_scale": 1},
        "default_chunk_size": 32 * 1024,
    }

    def build():
        model = transformers.BertForSequenceClassification(cfg)
        for p in list(model.bert.embeddings.parameters()) + list(model.bert.encoder.layer[0].parameters()):
            p.requires_grad_(False)
        return model

    engine, optimizer = ps.initialize_engine(model_func=build, local_rank=0, config=config)
    client, module = engine.client, engine.module
    cl, pos = client.chunk_list, client.positions()

    def snap(t):
        return t.detach().to("cpu", copy=True).numpy()

    mirror = [{"p32": snap(cl[q.fp32].payload), "m": snap(cl[q.exp_avg].payload), "v": snap(cl[q.exp_avg_sq].payload),
               "p16": snap(cl[q.fp16].payload)} for q in pos]
    oscaler = oracle.scaler_from_config(config["fp16"])
    oopt = oracle.OptimizerStepOracle(mirror, oscaler, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, use_adamw=True,
                                      tensors=tensor_spans(client, optimizer))
    n_head = len(oopt.tensors)
    ids = torch.randint(0, 256, (4, 32), device="cuda")
    labels = torch.randint(0, 2, (4,), device="cuda")
    kinds = []
    for it in range(9):
        if it == 3:
            for p in module.bert.encoder.layer[0].parameters():
                p.requires_grad_(True)
        if it == 5:
            for p in module.bert.embeddings.parameters():
                p.requires_grad_(True)
        oopt.tensors = tensor_spans(client, optimizer)
        poison = it == 6
        emb = module.bert.embeddings.word_embeddings.weight
        out = engine(input_ids=ids, labels=labels)
        loss = out.loss * (float("inf") if poison else 1.0)  # an overflowing loss: every gradient comes back inf / nan
        engine.backward(loss)
        for q, c in zip(pos, mirror):
            c["p16"][...] = snap(cl[q.fp16].payload)
        optimizer.step()
        kinds.append(optimizer._plan["kind"])
        oopt.check_overflow()
        assert oopt.step() == poison
        for i, (q, c) in enumerate(zip(pos, mirror)):
            for key, cid in (("p32", q.fp32), ("m", q.exp_avg), ("v", q.exp_avg_sq), ("p16", q.fp16)):
                assert_bits_equal(snap(cl[cid].payload), c[key], f"iteration {it} position {i} {key}")
        assert optimizer.loss_scaler.loss_scale == oscaler.loss_scale
    assert kinds == ["uniform"] * 3 + ["each"] * 6 and len(oopt.tensors) > n_head + 20
    head = module.classifier.weight
    layer0 = module.bert.encoder.layer[0].output.dense.weight
    assert [optimizer.state[p]["step"] for p in (head, layer0, emb)] == [8, 5, 3]
