"""Host side of models with per-sequence state: registry and configuration reader, state slots in the scheduler, steps
given from outside.  No device."""
import json

import pytest
import torch

from nano_vllm_x_amd.core.common import ForwardMode, SamplingParams, Sequence, SequenceStatus
from nano_vllm_x_amd.core.engine import EngineCore
from nano_vllm_x_amd.core.kv_cache import StateSlotAllocator
from nano_vllm_x_amd.core.scheduler import Scheduler

CFG = {"architecture": "Kabidra", "vocab": 40, "width": 16, "norm": {"eps": 1e-4}, "canon": {"taps": 3},
       "layers": [{"type": "mingru", "mixer": {"width": 24}, "mlp": None},
                  {"type": "latent_attention", "mixer": {"heads": 2, "dim": 8, "vdim": 4, "q_rank": 12, "kv_rank": 6, "scale": 0.5},
                   "mlp": {"kind": "dense", "ff": 20}}]}


def test_registry_reads_the_architecture_from_config_json(tmp_path):
    from nano_vllm_x_amd import registry
    from nano_vllm_x_amd.kabidra import KabidraConfig, KabidraForCausalLM
    from nano_vllm_x_amd.qwen3 import Qwen3Config, Qwen3ForCausalLM
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    cfg = registry.load_config(str(tmp_path))
    assert isinstance(cfg, KabidraConfig) and registry.model_class_of(cfg) is KabidraForCausalLM
    assert (cfg.vocab_size, cfg.width, cfg.eps, cfg.taps, len(cfg.layers)) == (40, 16, 1e-4, 3, 2)
    assert cfg.layers[1]["mixer"]["kv_rank"] == 6 and cfg.layers[0]["mlp"] is None
    q = tmp_path / "q"
    q.mkdir()
    (q / "config.json").write_text(json.dumps({"architectures": ["Qwen3ForCausalLM"], "hidden_size": 64, "num_attention_heads": 2,
                                               "num_key_value_heads": 1, "head_dim": 128, "num_hidden_layers": 1, "vocab_size": 50,
                                               "intermediate_size": 96}))
    cfg = registry.load_config(str(q))
    assert isinstance(cfg, Qwen3Config) and registry.model_class_of(cfg) is Qwen3ForCausalLM
    assert isinstance(registry.load_config("Qwen3-0.6B"), Qwen3Config)
    (q / "config.json").write_text(json.dumps({"architectures": ["SomethingElse"]}))
    with pytest.raises(ValueError):
        registry.load_config(str(q))


def test_configuration_refuses_what_the_design_does_not_have():
    from nano_vllm_x_amd.kabidra import KabidraConfig
    bad = json.loads(json.dumps(CFG))
    bad["layers"][0]["type"] = "lstm"
    with pytest.raises(ValueError):
        KabidraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CFG))
    bad["layers"][1]["mlp"]["kind"] = "experts"
    with pytest.raises(ValueError):
        KabidraConfig.from_dict(bad)


def test_checkpoint_names_and_state_shapes_follow_the_configuration():
    from nano_vllm_x_amd.kabidra import KabidraConfig, KabidraForCausalLM, checkpoint_shapes, random_checkpoint
    cfg = KabidraConfig.from_dict(CFG)
    shapes = checkpoint_shapes(cfg)
    assert shapes["l0.mix.z"] == (24, 16) and shapes["l1.mix.uk"] == (16, 6) and shapes["l1.mix.uv"] == (8, 6) and shapes["l1.dwa"] == (3,)
    assert "l0.norm2" not in shapes and "l0.canon2" not in shapes and "l1.canon2" in shapes
    model = KabidraForCausalLM(cfg)
    model.load_weights(random_checkpoint(cfg, 0))
    assert model.latent_ranks() == {1: 6}
    assert model.state_shapes() == {(0, "canon1"): (2, 16), (0, "gru"): (24,), (1, "canon1"): (2, 16), (1, "canon2"): (2, 16)}
    w = dict(random_checkpoint(cfg, 0))
    assert torch.equal(model.layers[0].mixer.zxg_proj.weight[24:48], w["l0.mix.x"].to(model.embed.dtype))
    assert torch.equal(model.layers[1].mixer.uv[1], w["l1.mix.uv"][4:8].to(model.embed.dtype))
    assert torch.equal(model.layers[1].mixer.down_proj.weight[18:20], w["l1.mix.g"].to(model.embed.dtype))


def test_state_slot_allocator_hands_out_the_lowest_free_slot():
    a = StateSlotAllocator(3)
    assert [a.alloc("x"), a.alloc("y"), a.alloc("z"), a.alloc("w")] == [0, 1, 2, None]
    assert a.alloc("y") == 1
    a.free("y")
    a.free("x")
    assert a.alloc("w") == 0 and a.num_free() == 1


def seq(i, n):
    return Sequence(seq_id=i, token_ids=list(range(n)), num_tokens=n, prompt_len=n)


def test_admission_waits_for_a_state_slot_and_finishing_returns_everything():
    s = Scheduler(kv_cache_size=100, max_bs=8, state_slots=2)
    for i, n in (("a", 5), ("b", 7), ("c", 3)):
        s.add_sequence(seq(i, n))
    batch = s.schedule()
    assert [x.seq_id for x in batch.seqs] == ["a", "b"] and [x.state_slot for x in batch.seqs] == [0, 1]
    for x in batch.seqs:
        s.update_sequence(x, 1)
    assert s.schedule().forward_mode == ForwardMode.DECODE      # c still waits: no slot
    s.finish_sequence(s.get_sequence("a"))
    # a model with state keeps no finished sequence's rows: they are free again at once
    assert s.kv_manager.kv_cache_allocator.num_free() == 100 - 8 and s.state_slots.num_free() == 1
    for x in list(s.running):
        s.scheduled.discard(x.seq_id)
    batch = s.schedule()
    assert [x.seq_id for x in batch.seqs] == ["c"] and batch.seqs[0].state_slot == 0
    with pytest.raises(ValueError):
        Scheduler(kv_cache_size=10, state_slots=2, prefix_reuse=True)


def test_preemption_gives_the_state_slot_back():
    s = Scheduler(kv_cache_size=15, max_bs=4, state_slots=3)
    for i, n in (("a", 5), ("b", 6), ("c", 4)):
        s.add_sequence(seq(i, n))
    for x in s.schedule().seqs:
        s.update_sequence(x, 1)
    batch = s.schedule()                      # the pool is full: the youngest sequence is preempted to let the others grow
    assert [x.seq_id for x in batch.seqs] == ["a", "b"]
    c = s.get_sequence("c")
    assert c.status == SequenceStatus.WAITING and c.state_slot is None and c.cached_kv_len == 0 and s.state_slots.num_free() == 1


def test_steps_given_from_outside_use_chunk_views_and_mixed_batches():
    core = EngineCore(kv_cache_size=64, max_bs=4, context_len=64, state_slots=4)
    core.add_sequence("a", [1, 2, 3, 4, 5], SamplingParams())
    core.add_sequence("b", [7], SamplingParams())
    sched = core.scheduler
    batch = sched.schedule_given([("a", 2), ("b", 1)])
    assert batch.forward_mode == ForwardMode.PREFILL
    view = batch.seqs[0]
    assert view.partial_of is sched.get_sequence("a") and view.token_ids == [1, 2] and view.state_slot == 0 and len(view.kv_indices) == 2
    with pytest.raises(RuntimeError):
        sched.schedule_given([("a", 1)])                      # already in flight
    sched.commit_given(batch)
    a = sched.get_sequence("a")
    assert a.cached_kv_len == 2 and sched.get_sequence("b").cached_kv_len == 1 and len(a.kv_indices) == 5
    core.extend_sequence("b", [8])
    batch = sched.schedule_given([("a", 3), ("b", 1)])        # the rest of a beside one more token of b
    assert batch.forward_mode == ForwardMode.PREFILL and batch.seqs[0] is a
    sched.commit_given(batch)
    core.extend_sequence("a", [6])
    core.extend_sequence("b", [9])
    batch = sched.schedule_given([("a", 1), ("b", 1)])
    assert batch.forward_mode == ForwardMode.DECODE            # every entry continues its sequence by one token
    sched.commit_given(batch)
    with pytest.raises(ValueError):
        sched.schedule_given([("a", 1)])                      # nothing waits
    core.abort_sequence("a")
    core.abort_sequence("b")
    assert sched.kv_manager.kv_cache_allocator.num_free() == 64 and sched.state_slots.num_free() == 4
    with pytest.raises(ValueError):
        core.add_sequence("c", [1], SamplingParams()) or core.extend_sequence("c", list(range(64)))


def test_oracle_convolution_and_recurrence_against_direct_formulas():
    """The restatement's own loops against closed forms on tiny inputs."""
    from oracle import kabidra_oracle as ko
    h = torch.arange(12.0).view(4, 3)
    k = torch.tensor([[1.0, 10.0], [2.0, 20.0], [0.0, 1.0]])      # taps = 2: k[:, 1] multiplies the current token
    out = ko.canon(h, k)
    assert torch.equal(out[0], h[0] + k[:, 1] * h[0]) and torch.equal(out[2], h[2] + k[:, 0] * h[1] + k[:, 1] * h[2])
    z, u, g = torch.zeros(3, 2), torch.tensor([[1.0, -50.0]] * 3), torch.full((3, 2), 50.0)
    y, s = ko.gru_scan(z, u, g)       # z = 1/2: S = 1.5 * (1 - 2^-t) for u = 1, and ~0 where the candidate is sigmoid(-50)
    assert torch.allclose(s, torch.tensor([1.5 * (1 - 0.125), 0.0]), atol=1e-6) and torch.allclose(y[:, 0], 50.0 * 1.5 * (1 - 0.5 ** torch.arange(1.0, 4.0)))
