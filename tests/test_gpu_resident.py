"""The device-resident target driver (ResidentTarget) under the speculative loop's own call
order (crates/itak-spec/src/session.rs:616-831): checkpoint(n + 1), one block forward over
[pending, drafts...], rewind to base + 1 + accepted, release, position check, note_spec_round,
round after round with seeded accept lengths, on a pool of sliding-window and global layers.

The model around the attention calls is a small seeded transformer whose other operators run
as torch matmuls in float64 (they are not this library's); every attention call goes through
the device step. The oracle replays what the device was given: for every block and layer the
q, k, v rows the model produced are appended to an oracle KvCache (with the reference's
checkpoint / rewind_to / release around the round) and attended on the CPU. Bars: attention
outputs within 2e-3, every layer's visible cache rows bit-exact at the end of every round."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import max_abs, pkg

pytestmark = pytest.mark.gpu

Q_HEADS, KV_HEADS, D, HIDDEN, VOCAB = 8, 2, 128, 64, 50


def P():
    return pkg()


class ToyLayers:
    """embed / qkv / mix / head over device tensors, recording what each attention call saw."""

    def __init__(self, layers, seed):
        g = torch.Generator(device="cpu").manual_seed(seed)

        def w(*shape, scale):
            return (torch.randn(*shape, generator=g, dtype=torch.float64) * scale).cuda()

        self.embed_table = w(VOCAB, HIDDEN, scale=1.0)
        self.wq = [w(HIDDEN, Q_HEADS * D, scale=HIDDEN ** -0.5) for _ in range(layers)]
        self.wk = [w(HIDDEN, KV_HEADS * D, scale=HIDDEN ** -0.5) for _ in range(layers)]
        self.wv = [w(HIDDEN, KV_HEADS * D, scale=HIDDEN ** -0.5) for _ in range(layers)]
        self.wo = [w(Q_HEADS * D, HIDDEN, scale=(Q_HEADS * D) ** -0.5) for _ in range(layers)]
        self.wout = w(HIDDEN, VOCAB, scale=HIDDEN ** -0.5)
        self.seen = []   # (layer, start_position, q, k, v) as numpy f32, in call order
        self.outs = []   # the attention outputs handed to mix, device tensors

    def embed(self, tokens):
        return self.embed_table[torch.as_tensor(list(tokens), device="cuda")]

    def qkv(self, layer, hidden, position):
        q = (hidden @ self.wq[layer]).float().contiguous()
        k = (hidden @ self.wk[layer]).float().contiguous()
        v = (hidden @ self.wv[layer]).float().contiguous()
        self.seen.append((layer, position, q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()))
        return q, k, v

    def mix(self, layer, hidden, attn_out):
        self.outs.append(attn_out)
        # Normalised residual stream: keeps Q and K at unit scale through the layers.
        h = hidden + torch.tanh(attn_out.double() @ self.wo[layer])
        return h / h.pow(2).mean(dim=-1, keepdim=True).sqrt()

    def head(self, hidden):
        return (hidden @ self.wout).float()


def check_blocks_against_oracle(toy, ref, first_call):
    """Replays the attention calls made since `first_call` on the oracle and compares."""
    worst = 0.0
    for (layer, position, q, k, v), out in zip(toy.seen[first_call:], toy.outs[first_call:]):
        want = oracle.attention_step(ref, layer, q, k, v, Q_HEADS, position, threads=4)
        worst = max(worst, max_abs(out.cpu().numpy().reshape(-1), want))
    return worst


def same_visible_rows(cache, ref, layers):
    for layer in range(layers):
        positions, rk, rv = ref.view(layer).rows()
        assert cache.next_position(layer) == ref.next_position(layer)
        assert cache.stored_len(layer) == len(positions)
        gp, gk, gv = cache.read_rows(layer, 0, len(positions))
        assert list(gp) == list(positions)
        assert np.array_equal(gk.reshape(len(positions), -1), oracle.f32_to_f16_array(rk).reshape(len(positions), -1))
        assert np.array_equal(gv.reshape(len(positions), -1), oracle.f32_to_f16_array(rv).reshape(len(positions), -1))


@pytest.mark.parametrize("seed", [0, 1])
def test_speculative_rounds_through_the_resident_driver(seed):
    W, G = P().LayerKind.windowed, P().LayerKind.Global
    window, depth = 96, 6
    pattern = [W(window), W(window), W(window), G] * 2   # the reference model's 3:1 pattern
    layers = len(pattern)
    pool = P().KvPool(pattern, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=1024,
                      ring_headroom=32)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    cache = pool.acquire()
    config = P().GlimmerConfig(layers=pattern, q_heads=Q_HEADS, kv_heads=KV_HEADS, key_length=D,
                               value_length=D, sliding_window=window)
    toy = ToyLayers(layers, seed)
    driver = P().ResidentTarget(pool, cache, config, toy, record_rounds=True)
    opattern = [oracle.LayerKind.windowed(window) if k.is_windowed else oracle.LayerKind.Global
                for k in pattern]
    ref = oracle.KvCache.new(opattern, KV_HEADS, D, store_f16=True)
    rng = np.random.default_rng(seed)

    # Prompt: chunks no longer than the rings' headroom, as the reference's session chunks them.
    prompt = rng.integers(0, VOCAB, size=150).tolist()
    calls = 0
    for at in range(0, len(prompt), 32):
        logits = driver.forward(prompt[at:at + 32])
        assert check_blocks_against_oracle(toy, ref, calls) <= 2e-3
        calls = len(toy.seen)
    assert driver.position() == len(prompt) == ref.next_position(0)
    same_visible_rows(cache, ref, layers)
    pending = int(torch.argmax(logits))

    emitted = []
    for round_no in range(12):
        base = driver.position()
        n = int(rng.integers(1, depth, endpoint=True))
        proposed = rng.integers(0, VOCAB, size=n).tolist()
        cp = driver.checkpoint(n + 1)
        ocp = ref.checkpoint(n + 1)
        block = [pending] + proposed
        logits, captures = driver.forward_block_capturing(block, [0, layers - 1])
        pool.synchronize()
        assert logits.shape == (n + 1, VOCAB) and [c.layer for c in captures] == [0, layers - 1]
        assert captures[0].rows.shape == (n + 1, HIDDEN)
        assert driver.position() == base + n + 1
        assert check_blocks_against_oracle(toy, ref, calls) <= 2e-3, round_no
        calls = len(toy.seen)
        accepted = int(rng.integers(0, n, endpoint=True))
        keep = base + 1 + accepted
        driver.rewind(cp, keep)
        driver.release(cp)
        ref.rewind_to(ocp, keep)
        ref.release(ocp)
        assert driver.position() == keep
        driver.note_spec_round(proposed, accepted)
        same_visible_rows(cache, ref, layers)
        # The correction token: the target's own choice at the first rejected (or bonus) row.
        pending = int(torch.argmax(logits[accepted]))
        emitted += proposed[:accepted] + [pending]
    records = driver.spec_round_records()
    assert len(records) == 12 and all(r.accepted <= r.proposed for r in records)
    assert driver.position() == len(prompt) + len(emitted)
    pool.close()


def test_resident_rewind_refusals_follow_the_session():
    W = P().LayerKind.windowed
    pattern = [W(64), P().LayerKind.Global]
    pool = P().KvPool(pattern, KV_HEADS, D, elem="f16", max_slots=1, capacity_rows=256,
                      ring_headroom=32)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    config = P().GlimmerConfig(layers=pattern, q_heads=Q_HEADS, kv_heads=KV_HEADS, key_length=D,
                               value_length=D, sliding_window=64)
    driver = P().ResidentTarget(pool, pool.acquire(), config, ToyLayers(2, 3))
    for _ in range(3):
        driver.forward([1] * 32)
    cp = driver.checkpoint(8)
    with pytest.raises(P().StepFailed) as e:   # session.rs:5398-5406
        driver.rewind(cp, 97)
    assert e.value.step == "session" and "ahead of the current position 96" in e.value.detail
    with pytest.raises(P().StepFailed) as e:   # session.rs:5407-5417
        driver.rewind(cp, 63)
    assert "discards 33 positions, past the 32-position ring headroom" in e.value.detail
    driver.rewind(cp, 64)
    driver.release(cp)
    assert driver.position() == 64
    with pytest.raises(P().StepFailed):
        driver.forward_block_capturing([1], [2])   # capture layer out of range
    assert driver.position() == 64
    driver.reset()
    assert driver.position() == 0
    driver.forward([2, 3])
    assert driver.position() == 2
    pool.close()


def _hybrid_target(seed, slots=1, softcap=0.0):
    W, G = P().LayerKind.windowed, P().LayerKind.Global
    pattern = [W(48), W(48), G, W(48)]
    pool = P().KvPool(pattern, KV_HEADS, D, elem="f16", max_slots=slots, capacity_rows=512,
                      ring_headroom=32)
    pool.set_stream(torch.cuda.current_stream().cuda_stream)
    config = P().GlimmerConfig(layers=pattern, q_heads=Q_HEADS, kv_heads=KV_HEADS, key_length=D,
                               value_length=D, sliding_window=48)
    return pool, config, pattern


def _view_bytes(cache, layers):
    out = []
    for layer in range(layers):
        n = cache.stored_len(layer)
        positions, k, v = cache.read_rows(layer, 0, n)
        out.append((list(positions), k.tobytes(), v.tobytes()))
    return out


@pytest.mark.parametrize("elem", ["f32", "f16"])
def test_forward_with_prefix_store_cold_partial_and_full_hits(tmp_path, monkeypatch, capfd, elem):
    # ResidentSession::forward_with_prefix_store (crates/wgpu-compute/src/session.rs:5122-5151)
    # on a hybrid pool. Chunks are 48 rows here (what the rings hold beyond their window), and the prompts are cut so
    # that a run that restores a prefix makes the same launches over the same rows as the cold
    # run it is compared with: logits and stored rows are then equal bit for bit, which is the
    # reference's claim for its own chunking ("reproduces exactly the cold run's last step").
    monkeypatch.setenv("ITAK_KV_PREFIX_STORE", "1")
    rng = np.random.default_rng(77)
    tokens = rng.integers(0, VOCAB, size=146).tolist()
    fp = "toy-model"
    pool, config, pattern = _hybrid_target(5, slots=6)
    layers = len(pattern)

    def target():
        return P().ResidentTarget(pool, pool.acquire(), config, ToyLayers(layers, 5))

    # A prompt of 97 tokens = chunks of 48, 48 and 1: cold (a miss that files the prefix), then
    # the same prompt again: a hit over the whole prompt, rewound by one, the last token
    # forwarded again.
    store = P().PrefixStore.open(str(tmp_path / "one"), 1 << 30)
    cold = target()
    cold_logits = cold.forward_with_prefix_store(store, tokens[:97], fp, elem=elem)
    assert cold.position() == 97 and store.stats().entries == 1
    assert store.entries()[0].token_count == 97
    full = target()
    full_logits = full.forward_with_prefix_store(store, tokens[:97], fp, elem=elem)
    assert full.position() == 97
    assert len(full._layers.seen) == layers  # one block of one row per layer, nothing else
    assert all(rows.shape[0] == 1 and pos == 96 for _, pos, rows, _, _ in full._layers.seen)
    assert torch.equal(full_logits, cold_logits)
    assert _view_bytes(full._cache, layers) == _view_bytes(cold._cache, layers)

    # A stored prefix of 96 tokens under a prompt of 144: the rest is one chunk of 48, as the
    # cold run's third chunk is.
    store2 = P().PrefixStore.open(str(tmp_path / "two"), 1 << 30)
    first = target()
    first.forward_with_prefix_store(store2, tokens[:96], fp, elem=elem)
    assert store2.entries()[0].token_count == 96
    partial = target()
    partial_logits = partial.forward_with_prefix_store(store2, tokens[:144], fp, elem=elem)
    assert partial.position() == 144
    assert [pos for _, pos, _, _, _ in partial._layers.seen] == [96] * layers
    assert sorted(e.token_count for e in store2.entries()) == [96, 144]  # hit or miss, the whole prefix is filed
    monkeypatch.setenv("ITAK_KV_PREFIX_STORE", "0")   # the switch off: exactly forward
    plain = target()
    plain_logits = plain.forward_with_prefix_store(store2, tokens[:144], fp, elem=elem)
    assert len(store2.entries()) == 2
    assert torch.equal(partial_logits, plain_logits)
    assert _view_bytes(partial._cache, layers) == _view_bytes(plain._cache, layers)
    monkeypatch.setenv("ITAK_KV_PREFIX_STORE", "1")

    # Mid-sequence the store is not consulted and nothing is filed.
    entries = len(store2.entries())
    more = partial.forward_with_prefix_store(store2, tokens[144:145], fp, elem=elem)
    assert partial.position() == 145 and len(store2.entries()) == entries and more.shape == (VOCAB,)

    # A store whose directory has gone (a file stands in its place): the lookup is refused, the
    # cold prefill serves, the capture fails, and the forward's result stands; the failure is
    # named on the diagnostic channel.
    root = tmp_path / "three"
    store3 = P().PrefixStore.open(str(root), 1 << 30)
    os.rmdir(root)
    root.write_text("not a directory")
    P().set_debug_enabled(True)
    capfd.readouterr()
    try:
        broken = target()
        broken_logits = broken.forward_with_prefix_store(store3, tokens[:97], fp, elem=elem)
    finally:
        P().set_debug_enabled(False)
    assert torch.equal(broken_logits, cold_logits)
    assert "post-forward capture/store failed" in capfd.readouterr().err
    pool.close()
