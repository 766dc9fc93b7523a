"""Host-side parts of the Puguzen family that need no GPU: the configuration reader and model
registry, the slot and page bookkeeping, and the plain CPU model's own consistency (a prompt fed
whole, in portions, or token by token gives the same logits; the visibility rule of the windowed
layer against its definition)."""
import json
import os
import subprocess

import pytest
import torch

from oracle import puguzen as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CFG = {"architecture": "Puguzen", "width": 48, "vocab": 70, "norm": {"eps": 1e-6}, "layers": [
    {"type": "retention", "mixer": {"heads": 2, "dim": 12, "vdim": 8, "decay": [0.9, 0.99],
                                    "rot": {"dims": 8, "base": 100.0}}, "mlp": {"kind": "dense", "ff": 40}},
    {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "scale": 0.5,
                                    "rot": {"dims": 8, "base": 777.0}, "mask": {"size": 6, "pool": 3}}, "mlp": None},
    {"type": "gla", "mixer": {"heads": 3, "dim": 8, "vdim": 8, "tau": 4.0}, "mlp": {"kind": "dense", "ff": 24}},
]}


def test_visible_keys_is_the_definition():
    for size in (1, 2, 5, 8):
        for pool in (1, 2, 3, 8):
            for i in range(40):
                toks, blocks = P.visible_keys(i, size, pool)
                assert toks == [j for j in range(i + 1) if 0 <= i - j < size]
                assert blocks == [b for b in range(i + 1) if b * pool + pool - 1 <= i - size]
                # a token is never seen twice
                assert not set(toks) & {j for b in blocks for j in range(b * pool, b * pool + pool)}


def test_plain_model_does_not_care_how_a_prompt_is_cut():
    st = P.random_model(CFG, 1)
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, CFG["vocab"], (45,), generator=g).tolist()
    whole = P.forward(CFG, st, toks, P.Sequence(CFG))
    for cuts in ([1] * 45, [2, 7, 1, 20, 15], [44, 1]):
        seq, got, at = P.Sequence(CFG), [], 0
        for c in cuts:
            got.append(P.forward(CFG, st, toks[at:at + c], seq))
            at += c
        assert torch.allclose(torch.cat(got), whole, atol=1e-10, rtol=0)


def test_config_reader_and_registry(tmp_path):
    from safetensors.torch import save_file
    from vllm_omni_draft_amd import config
    st = P.random_model(CFG, 2)
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    save_file({k: v.to(torch.bfloat16) for k, v in st.items()}, str(tmp_path / "model.safetensors"))
    mc = config.load_model_config(str(tmp_path))
    assert isinstance(mc, config.SeqModelConfig) and mc.n_layers == 3 and mc.width == 48 and mc.norm_eps == 1e-6
    r, a, g = (l.mixer for l in mc.layers)
    assert (r.kind, r.rot_dims, r.rot_layout, r.decay, r.kv_heads) == ("retention", 8, "half", (0.9, 0.99), 2)
    assert (a.kind, a.kv_heads, a.window, a.pool, a.scale, a.rot_layout, a.rot_base) == \
        ("attention", 2, 6, 3, 0.5, "interleaved", 777.0)
    assert (g.kind, g.tau, g.rank) == ("gla", 4.0, st["l2.mix.a1"].shape[0])      # the rank comes from a tensor
    assert [l.ff for l in mc.layers] == [40, 0, 24]
    assert mc.state_bytes_per_seq() == 4 * (2 * 12 * 8 + 3 * 8 * 8)
    # a Hugging Face decoder still goes the other way
    (tmp_path / "config.json").write_text(json.dumps({
        "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 2,
        "intermediate_size": 256, "vocab_size": 256}))
    assert isinstance(config.load_model_config(str(tmp_path)), config.ModelConfig)
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Nope"}))
    with pytest.raises(ValueError):
        config.load_model_config(str(tmp_path))


@pytest.mark.parametrize("bad", [
    {"type": "attention", "mixer": {"heads": 4, "kv_heads": 3, "dim": 8, "vdim": 8, "mask": {"size": 4, "pool": 2}}},
    {"type": "attention", "mixer": {"heads": 2, "dim": 8, "vdim": 8, "mask": {"size": 0, "pool": 2}}},
    {"type": "retention", "mixer": {"heads": 2, "dim": 8, "vdim": 8, "decay": [0.5]}},
    {"type": "retention", "mixer": {"heads": 1, "dim": 8, "vdim": 8, "decay": [0.5], "rot": {"dims": 10, "base": 10.0}}},
    {"type": "gla", "mixer": {"heads": 1, "dim": 8, "vdim": 8, "tau": 0.0}},
    {"type": "conv", "mixer": {"heads": 1, "dim": 8, "vdim": 8}},
])
def test_config_reader_refuses(bad):
    from vllm_omni_draft_amd import config
    cfg = dict(CFG, layers=[dict(bad, mlp=None)])
    with pytest.raises(ValueError):
        config.puguzen_config(cfg)


def test_slot_and_page_bookkeeping():
    from vllm_omni_draft_amd import _lib, config
    from vllm_omni_draft_amd.kv_cache import PAGE, OutOfPages, OutOfSlots, SeqCache
    if not os.path.exists(_lib.lib_path()):
        subprocess.run(["make", "-C", ROOT, "-j8"], check=True)
    st = P.random_model(CFG, 2)
    mc = config.puguzen_config(CFG, {k: tuple(v.shape) for k, v in st.items()})
    c = SeqCache(mc, torch.float32, max_seqs=2, num_pages=5, max_seq_len=4 * PAGE, device="cpu")
    assert sorted(c.state) == [0, 2] and sorted(c.k) == [1] and c.state[0].shape == (2, 2, 12, 8)
    assert c.pk[1].shape[2] >= PAGE // 3 + 1
    a, b = c.slots.alloc(), c.slots.alloc()
    with pytest.raises(OutOfSlots):
        c.slots.alloc()
    c.ensure_capacity(a, PAGE + 1)
    c.ensure_capacity(b, 3 * PAGE)
    assert len(c.pages_of(a)) == 2 and len(c.pages_of(b)) == 3 and c.allocator.num_free == 0
    assert c.block_tables[a, :2].tolist() == c.pages_of(a)
    with pytest.raises(OutOfPages):
        c.ensure_capacity(a, 2 * PAGE + 1)          # the pool is empty
    assert len(c.pages_of(a)) == 2                   # and a refused request took nothing
    with pytest.raises(OutOfPages):
        c.ensure_capacity(b, 4 * PAGE + 1)          # longer than max_seq_len
    freed = set(c.pages_of(b))
    c.release(b)
    assert c.allocator.num_free == 3 and c.slots.num_free == 1
    b2 = c.slots.alloc()
    c.ensure_capacity(b2, 2 * PAGE)
    assert set(c.pages_of(b2)) <= freed              # pages come back into use
    with pytest.raises(ValueError):
        c.slots.free(5) or c.slots.free(5)
