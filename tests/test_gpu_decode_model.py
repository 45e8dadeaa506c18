"""The decode-step module (prefill + captured decode step) on a small text-tower configuration
against the CPU restatement of the same op sequence (oracle/decode_step.py).

Logits are FLOAT32; tolerance 2e-3 absolute (fp16 data formats inside the step: weights, the
activation entering each Linear, q and the KV cache)."""
import numpy as np
import pytest

from axono_amd import DataType, Tensor
from axono_amd.examples.qwen3vl_text import Qwen3VLTextDecoder, TextConfig, random_weights
from oracle.decode_step import OracleDecoder

pytestmark = pytest.mark.gpu

CFG = TextConfig(num_hidden_layers=3, hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
                 intermediate_size=512, vocab_size=1000)


# four query heads per kv head: decode attention (and its decode-step form) on the matrix cores
CFG4 = TextConfig(num_hidden_layers=2, hidden_size=256, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
                  intermediate_size=512, vocab_size=1000)


# the small widths the fused layer launch is built for (hidden 512 = 4 heads of 128, intermediate 1024, 4 + 2 * 2 heads
# of q / k / v): every layer but the last runs behind its attention as one persistent launch
CFG_FUSED = TextConfig(num_hidden_layers=4, hidden_size=512, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
                       intermediate_size=1024, vocab_size=1000)


def _setup(B=3, S=21, max_len=64, seed=0, CFG=CFG):
    w = random_weights(CFG, seed)
    # non-trivial norm weights so a dropped weight would show
    rng = np.random.default_rng(seed + 1)
    for k in w:
        if k.endswith("norm.weight") or k.endswith("layernorm.weight"):
            w[k] = (1 + 0.1 * rng.standard_normal(w[k].shape)).astype(np.float32)
    gpu = Qwen3VLTextDecoder(CFG, w, B, max_len, "hip:0")
    cpu = OracleDecoder(CFG, w, B, max_len)
    ids = rng.integers(0, CFG.vocab_size, (B, S)).astype(np.int64)
    return gpu, cpu, ids



def assert_cache_rows(got, want, layer, fp32_term=1e-4):
    """Cache rows (fp16) of the device against the restatement's: both sides round an fp32 value once, so they are
    equal or neighbours wherever those fp32 values agree to within `fp32_term`.  What that term has to cover at
    layer 0 (identical residual stream): the activation entering the qkv Linear is stored as fp16 on both sides, an
    fp32 last-bit difference flips a few of its 256 elements by one fp16 ulp (1e-3 * |w| = 2e-5 each in the Linear
    output), and the k-norm divides by the head's rms (0.3 at this width), which carries up to 2.5e-4 into k - hence
    5e-4 for k and 1e-4 for v.  Deeper layers of a free-running comparison see a residual stream that already
    differs by such flips; for them the bound is two fp16 steps at |v| < 4 (4e-3), and the layer-wise tests compare
    every layer on identical inputs."""
    got, want = got.astype(np.float32), want.astype(np.float32)
    err = np.abs(got - want)
    if layer > 0:
        assert err.max() <= 4e-3, (layer, float(err.max()))
        return
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float32)
    assert np.all(err <= ulp + fp32_term), (layer, float(err.max()), float((err - ulp).max()))
    assert np.mean(err > 0) <= 0.2, float(np.mean(err > 0))


def test_prefill_logits_and_cache():
    gpu, cpu, ids = _setup()
    g_logits, g_next = gpu.prefill(ids)
    c_logits, c_next = cpu.prefill(ids)
    err = np.abs(g_logits.to_numpy() - c_logits).max()
    assert err <= 2e-3, err
    S = ids.shape[1]
    for i in range(CFG.num_hidden_layers):
        kc, vc = gpu.cache.get(i)
        assert_cache_rows(kc.numpy()[:, :, :S], cpu.k[i][:, :, :S], i, 5e-4)
        assert_cache_rows(vc.numpy()[:, :, :S], cpu.v[i][:, :, :S], i)
        assert np.all(kc.numpy()[:, :, S:] == 0)
    np.testing.assert_array_equal(gpu.cache.seq_lens.to_numpy(), [S] * ids.shape[0])


@pytest.mark.parametrize("use_graph", [False, True])
def test_decode_steps_match_oracle(use_graph):
    gpu, cpu, ids = _setup(seed=3)
    B, S = ids.shape
    _, g_next = gpu.prefill(ids)
    _, c_next = cpu.prefill(ids)
    first = g_next.to_numpy()
    pos = np.full((3, B), S, np.int64)  # text-only: position = index of the token being decoded
    n_steps = 6
    gpu.start_decode(first, pos, n_steps)
    if use_graph:
        g = gpu.capture()
        assert g.num_nodes > 10
    toks = gpu.generate(n_steps, use_graph=use_graph)
    # the oracle follows the GPU's token choices so that one near-tie cannot derail the comparison
    cur = first
    for s in range(n_steps):
        logits, nxt = cpu.decode_step(cur, pos + s)
        # the GPU token must be (within tolerance) a maximiser of the oracle's logits
        chosen = logits[np.arange(B), toks[s]]
        assert np.all(chosen >= logits.max(-1) - 4e-3), (s, chosen, logits.max(-1))
        cur = toks[s]
    np.testing.assert_array_equal(gpu.cache.seq_lens.to_numpy(), [S + n_steps] * B)
    # cache rows written by the decode steps
    for i in range(CFG.num_hidden_layers):
        assert_cache_rows(gpu.cache.get(i)[0].numpy()[:, :, S:S + n_steps], cpu.k[i][:, :, S:S + n_steps], i, 5e-4)


@pytest.mark.parametrize("use_graph", [False, True])
def test_decode_steps_with_the_fused_layer_launch_match_oracle(use_graph):
    """The same comparison at widths the fused layer launch is built for: three such launches per step hand the
    residual stream and the next q/k/v projection to each other, the fourth layer's closes with the final norm; three
    sequences (rows 3 to 15 of the launch's 16 are unused), eager and captured; and the tokens equal those of the
    same model run as single operators."""
    from axono_amd import libaxono as L
    gpu, cpu, ids = _setup(seed=11, CFG=CFG_FUSED)
    assert gpu._fused_tail
    B, S = ids.shape
    _, g_next = gpu.prefill(ids)
    cpu.prefill(ids)
    first = g_next.to_numpy()
    pos = np.full((3, B), S, np.int64)
    n_steps = 6
    gpu.start_decode(first, pos, n_steps)
    if use_graph:
        g = gpu.capture()
        # embedding + first norm, first q/k/v, (attention, fused launch) x 4, lm_head, argmax, state advance
        assert g.num_nodes == 2 + 2 * 4 + 3
    toks = gpu.generate(n_steps, use_graph=use_graph)
    assert L.decode_layer_tail_failed_waits() == 0
    cur = first
    for s in range(n_steps):
        logits, _ = cpu.decode_step(cur, pos + s)
        chosen = logits[np.arange(B), toks[s]]
        assert np.all(chosen >= logits.max(-1) - 4e-3), (s, chosen, logits.max(-1))
        cur = toks[s]
    np.testing.assert_array_equal(gpu.cache.seq_lens.to_numpy(), [S + n_steps] * B)
    for i in range(CFG_FUSED.num_hidden_layers):
        assert_cache_rows(gpu.cache.get(i)[0].numpy()[:, :, S:S + n_steps], cpu.k[i][:, :, S:S + n_steps], i, 5e-4)

    # the same model as single operators
    w = random_weights(CFG_FUSED, 11)
    rng = np.random.default_rng(12)
    for k in w:
        if k.endswith("norm.weight") or k.endswith("layernorm.weight"):
            w[k] = (1 + 0.1 * rng.standard_normal(w[k].shape)).astype(np.float32)
    plain = Qwen3VLTextDecoder(CFG_FUSED, w, B, 64, "hip:0", fused_tail=False)
    _, p_next = plain.prefill(ids)
    np.testing.assert_array_equal(p_next.to_numpy(), first)
    plain.start_decode(first, pos, n_steps)
    if use_graph:
        plain.capture()
    toks_plain = plain.generate(n_steps, use_graph=use_graph)
    cur = first
    for s in range(n_steps):   # (a near-tie may be broken differently: both must be maximisers for the oracle)
        if not np.array_equal(toks_plain[s], toks[s]):
            logits, _ = cpu.decode_step(cur, pos + s)
            break
        cur = toks[s]
    else:
        return
    chosen = logits[np.arange(B), toks_plain[s]]
    assert np.all(chosen >= logits.max(-1) - 4e-3)


def test_compiled_decode_loop_matches_the_captured_step():
    """The reference's loop shape (examples/vlm/qwen3vl/model.py:827-861) over `axono.compile(model)`:
    every step refreshes ids / positions in place, replays, and advances the cache from the host side.
    Same tokens as the device-driven captured step."""
    import axono_amd as axono
    n_steps = 5
    gpu, _, ids = _setup(seed=5)
    B, S = ids.shape
    _, g_next = gpu.prefill(ids)
    first = g_next.to_numpy().copy()
    gpu.start_decode(first, np.full((3, B), S, np.int64), n_steps)
    gpu.capture()
    want = gpu.generate(n_steps)

    gpu2, _, _ = _setup(seed=5)
    gpu2.prefill(ids)
    compiled = axono.compile(gpu2)
    cur = Tensor(DataType.INT64, [B], "hip:0")
    pos = Tensor(DataType.INT64, [3, B], "hip:0")
    tok = first
    got = []
    for s in range(n_steps):
        cur.copy_from_numpy(tok)
        pos.copy_from_numpy(np.full((3, B), S + s, np.int64))
        logits, nxt = compiled(cur, pos)
        tok = nxt.to_numpy().copy()
        got.append(tok)
        gpu2.cache.advance(1)
    np.testing.assert_array_equal(np.stack(got), want)
    np.testing.assert_array_equal(gpu2.cache.seq_lens.to_numpy(), [S + n_steps] * B)
    assert len(compiled._graphs) == 1


def test_eager_and_graph_logits_agree_every_replay():
    """Each replay is checked against an eager run of the same step from the same state."""
    gpu, _, ids = _setup(seed=7)
    B, S = ids.shape
    _, nxt = gpu.prefill(ids)
    first = nxt.to_numpy()
    pos = np.full((3, B), S, np.int64)
    gpu.start_decode(first, pos, 8)
    gpu.capture()
    for s in range(4):
        state = (gpu._ids.numpy().copy(), gpu._pos.numpy().copy(), gpu.cache.seq_lens.numpy().copy())
        e_logits, e_next = gpu._step_fn()
        e_logits, e_next = e_logits.to_numpy().copy(), e_next.to_numpy().copy()
        gpu._ids.copy_from_numpy(state[0])
        gpu._pos.copy_from_numpy(state[1])
        gpu.cache.seq_lens.copy_from_numpy(state[2])
        gpu._graph.replay()
        np.testing.assert_array_equal(gpu._graph_out[0].to_numpy(), e_logits)
        np.testing.assert_array_equal(gpu._graph_out[1].to_numpy(), e_next)


def test_decode_steps_match_oracle_with_four_heads_per_kv_head():
    """The captured step of a model whose attention runs on the matrix-core decode path (group size 4)."""
    gpu, cpu, ids = _setup(seed=11, CFG=CFG4)
    B, S = ids.shape
    g_logits, g_next = gpu.prefill(ids)
    c_logits, _ = cpu.prefill(ids)
    assert np.abs(g_logits.to_numpy() - c_logits).max() <= 2e-3
    first = g_next.to_numpy()
    pos = np.full((3, B), S, np.int64)
    n_steps = 5
    gpu.start_decode(first, pos, n_steps)
    gpu.capture()
    toks = gpu.generate(n_steps, use_graph=True)
    cur = first
    for s in range(n_steps):
        logits, _ = cpu.decode_step(cur, pos + s)
        chosen = logits[np.arange(B), toks[s]]
        assert np.all(chosen >= logits.max(-1) - 4e-3), (s, chosen, logits.max(-1))
        cur = toks[s]
    for i in range(CFG4.num_hidden_layers):
        kc, vc = gpu.cache.get(i)
        n = S + n_steps
        assert_cache_rows(kc.numpy()[:, :, :n], cpu.k[i][:, :, :n], i, 5e-4)
        assert_cache_rows(vc.numpy()[:, :, :n], cpu.v[i][:, :, :n], i)


def test_generate_refuses_to_run_past_the_bound_the_step_was_captured_for():
    gpu, _, ids = _setup(seed=13, max_len=40)
    B, S = ids.shape
    _, nxt = gpu.prefill(ids)
    gpu.start_decode(nxt.to_numpy(), np.full((3, B), S, np.int64), 4)
    gpu.capture()
    gpu.generate(4)
    with pytest.raises(RuntimeError, match="start_decode"):
        gpu.generate(4)                      # 21 + 4 + 4 > the bound of 26 the step was captured for
    gpu.start_decode(gpu._ids.numpy(), gpu._pos.numpy(), 15)
    gpu.capture()
    gpu.generate(15)                         # fills the cache to its 40 positions
    gpu.start_decode(gpu._ids.numpy(), gpu._pos.numpy(), 1)
    with pytest.raises(RuntimeError, match="full"):
        gpu.generate(1)


def test_device_is_no_farther_from_the_float64_evaluation_than_the_fp32_restatement():
    """Two correct fp32 pipelines drift apart at the fp16 storage points of a decode step (a 1e-7 difference
    can round to the other fp16 neighbour).  The yardstick is the same op sequence in float64 with the
    same storage points (oracle/f64_ops.py): over several decode steps from identical caches, the
    device's logits are no farther from it than 1.5 x the fp32 restatement's are (with a floor of one
    fp16 flip's worth), and each layer evaluated from the device's own input to that layer stays within
    2e-3 of both."""
    from oracle.f64_ops import F64Ops

    gpu, cpu32, ids = _setup(seed=17)
    cfg = CFG
    B, S = ids.shape
    _, g_next = gpu.prefill(ids)
    cpu64 = OracleDecoder(cfg, cpu32.w, B, gpu.cache.max_len, ops=F64Ops())

    def sync_caches(n):
        for i in range(cfg.num_hidden_layers):
            kc, vc = gpu.cache.get(i)
            for c in (cpu32, cpu64):
                c.k[i][:] = kc.numpy()
                c.v[i][:] = vc.numpy()
        cpu32.lens[:] = n
        cpu64.lens[:] = n

    cur = g_next.to_numpy().copy()
    d_gpu, d_cpu, layer_gpu, layer_cpu = 0.0, 0.0, 0.0, 0.0
    for s in range(4):
        n = S + s
        sync_caches(n)
        pos = np.full((3, B), n, np.int64)
        idt, post = Tensor(DataType.INT64, [B], "hip:0"), Tensor(DataType.INT64, [3, B], "hip:0")
        idt.copy_from_numpy(cur)
        post.copy_from_numpy(pos)
        trace = []
        g_logits, g_tok = gpu.decode_forward(idt, post, trace=trace)
        g_logits, g_tok = g_logits.to_numpy().copy(), g_tok.to_numpy().copy()
        h_gpu = [t.to_numpy().copy() for t in trace]
        l64, _ = cpu64.decode_step(cur, pos)
        l32, _ = cpu32.decode_step(cur, pos)
        d_gpu = max(d_gpu, float(np.abs(g_logits - l64).max()))
        d_cpu = max(d_cpu, float(np.abs(l32 - l64).max()))
        # layer by layer from the device's own inputs
        cpu32.lens[:] = n
        cpu64.lens[:] = n
        o64, _ = cpu64.decode_layers_teacher_forced(h_gpu, pos)
        o32, _ = cpu32.decode_layers_teacher_forced(h_gpu, pos)
        for i in range(cfg.num_hidden_layers):
            layer_gpu = max(layer_gpu, float(np.abs(h_gpu[i + 1] - o64[i]).max()))
            layer_cpu = max(layer_cpu, float(np.abs(o32[i] - o64[i]).max()))
        gpu.cache.advance(1)
        cur = g_tok
    assert d_gpu <= max(1.5 * d_cpu, 1e-3), (d_gpu, d_cpu)
    assert layer_gpu <= 2e-3 and layer_cpu <= 2e-3, (layer_gpu, layer_cpu)
    assert layer_gpu <= max(1.5 * layer_cpu, 1e-3), (layer_gpu, layer_cpu)


def test_paged_decoder_gives_the_tokens_and_logits_of_the_dense_one():
    """The decoder over a PagedKVCache (prefill through a dense scratch block copied into pages, decode step
    with the paged attention launch, captured and replayed) against the same decoder over the static cache:
    same prefill logits, same tokens, same logits of the last replay, bit for bit; pages in use follow the
    tokens; and against the oracle like the dense one."""
    n_steps = 6
    dense, cpu, ids = _setup(seed=23, S=125, max_len=160)      # the steps cross the first page boundary
    B, S = ids.shape
    w = cpu.w
    paged = Qwen3VLTextDecoder(CFG, w, B, 160, "hip:0", paged=True)
    outs = {}
    for name, m in (("dense", dense), ("paged", paged)):
        logits, nxt = m.prefill(ids)
        first = nxt.to_numpy().copy()
        m.start_decode(first, np.full((3, B), S, np.int64), n_steps)
        m.capture()
        toks = m.generate(n_steps)
        outs[name] = (logits.to_numpy().copy(), first, toks, m._graph_out[0].to_numpy().copy())
    for a, b in zip(outs["dense"], outs["paged"]):
        np.testing.assert_array_equal(a, b)
    assert paged.cache.pages_in_use == B * 2 and len(paged.cache) == S + n_steps
    np.testing.assert_array_equal(paged.cache.seq_lens.to_numpy(), [S + n_steps] * B)
    # the cached rows, read back through the page table, are the dense cache's rows
    table = paged.cache.page_table.to_numpy()
    for i in range(CFG.num_hidden_layers):
        kd = dense.cache.get(i)[0].numpy()
        kp = paged.cache.get(i)[0].numpy()
        for b in range(B):
            for pg in range(2):
                rows = min(128, S + n_steps - pg * 128)
                np.testing.assert_array_equal(kp[table[b, pg], :, :rows].view(np.uint16),
                                              kd[b, :, pg * 128:pg * 128 + rows].view(np.uint16))
    # and the oracle accepts the tokens
    c_logits, _ = cpu.prefill(ids)
    assert np.abs(outs["paged"][0] - c_logits).max() <= 2e-3
    cur, pos = outs["paged"][1], np.full((3, B), S, np.int64)
    for s in range(n_steps):
        logits, _ = cpu.decode_step(cur, pos + s)
        chosen = logits[np.arange(B), outs["paged"][2][s]]
        assert np.all(chosen >= logits.max(-1) - 4e-3)
        cur = outs["paged"][2][s]


@pytest.mark.parametrize("paged", [False, True])
def test_one_dealing_of_the_key_ranges_per_step_changes_no_bit(paged):
    """The captured step whose attention launches of layers 1.. take their key ranges from the table layer 0's launch
    leaves (the default) against the same model with every launch dealing for itself: same tokens and the same logits
    of the last replay, bit for bit, over replays in which the lengths grow (ragged start: prefill of the longest,
    then the lengths set by hand), dense and paged."""
    n_steps = 7
    shared, cpu, ids = _setup(seed=29, S=100, max_len=160)
    B, S = ids.shape
    each = Qwen3VLTextDecoder(CFG, cpu.w, B, 160, "hip:0", paged=paged, plan_reuse=False)
    if paged:
        shared = Qwen3VLTextDecoder(CFG, cpu.w, B, 160, "hip:0", paged=True)
    assert shared._plan_reuse and not each._plan_reuse
    outs = []
    for m in (shared, each):
        _, nxt = m.prefill(ids)
        first = nxt.to_numpy().copy()
        # sequences of different lengths: the rows beyond a sequence's length stay in the cache and are not attended
        lens = np.array([S, S - 37, 5][:B], np.int32)
        m.cache.set_lengths(lens)
        m.start_decode(first, np.tile(lens.astype(np.int64), (3, 1)), n_steps)
        m.capture()
        toks = m.generate(n_steps)
        outs.append((toks, m._graph_out[0].to_numpy().copy(), m.cache.seq_lens.to_numpy().copy()))
    for a, b in zip(*outs):
        np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(outs[0][2], [S + n_steps, S - 37 + n_steps, 5 + n_steps][:B])


@pytest.mark.parametrize("fused_tail,n_layers", [(False, 2), (True, 3)])
def test_captured_step_at_the_real_widths_of_the_2b_shape(fused_tail, n_layers):
    """The launches of the benchmark's decode step at their real sizes, two or three layers deep (three with the
    part of a layer behind its attention as one persistent launch: two such launches in a row share the workspace
    and hand the residual stream and the q/k/v projection on, the last layer runs as single operators): hidden 2048, 16 / 8 heads of
    128, intermediate 6144 (gate+up 2048 -> 12288 with three row tiles per workgroup and the SiLU-mul epilogue),
    vocabulary 151 936 (lm_head + the wide argmax), batch 16, caches filled with seeded random fp16 rows to 4096
    keys (attention cuts every sequence into two ranges merged by ticket; no prefill).  One replay of the captured
    step against the restatement: every layer from the device's own input to it (<= 2e-3), logits from the
    device's final state (<= 2e-3), cache rows of the new token, device-side argmax, advanced lengths; a second
    replay must be accepted by the oracle run free from the first one's token."""
    import time

    t_start = time.perf_counter()
    cfg = TextConfig(num_hidden_layers=n_layers)
    B, ctx, max_len, n_steps = 16, 4096, 4224, 2
    w = random_weights(cfg, 41)
    rng = np.random.default_rng(42)
    for k in w:
        if k.endswith("norm.weight") or k.endswith("layernorm.weight"):
            w[k] = (1 + 0.1 * rng.standard_normal(w[k].shape)).astype(np.float32)
    gpu = Qwen3VLTextDecoder(cfg, w, B, max_len, "hip:0", fused_tail=fused_tail)
    cpu = OracleDecoder(cfg, w, B, max_len)
    nkv, D = cfg.num_key_value_heads, cfg.head_dim
    for i in range(cfg.num_hidden_layers):
        # keys as the k-norm leaves them (unit rms per row), values like a projection output
        kk = np.zeros((B, nkv, max_len, D), np.float16)
        vv = np.zeros((B, nkv, max_len, D), np.float16)
        kk[:, :, :ctx] = rng.standard_normal((B, nkv, ctx, D), dtype=np.float32).astype(np.float16)
        vv[:, :, :ctx] = (0.7 * rng.standard_normal((B, nkv, ctx, D), dtype=np.float32)).astype(np.float16)
        kc, vc = gpu.cache.get(i)
        kc.copy_from_numpy(kk)
        vc.copy_from_numpy(vv)
        cpu.k[i][:] = kk
        cpu.v[i][:] = vv
    gpu.cache.set_lengths(np.full(B, ctx, np.int32))
    cpu.lens[:] = ctx
    first = rng.integers(0, cfg.vocab_size, B).astype(np.int64)
    pos = np.stack([np.full(B, ctx), rng.integers(0, ctx, B), rng.integers(0, ctx, B)]).astype(np.int64)  # t, h, w differ
    trace = []
    gpu.start_decode(first, pos, n_steps, trace=trace)
    g = gpu.capture()
    # single operators: 7 launches per layer; fused: attention + one launch per layer but the last, whose q/k/v
    # projection the launch before it has already run
    # fused: embedding + first norm, first q/k/v, (attention, fused launch) per layer, lm_head, argmax, state advance
    assert g.num_nodes == (2 + 2 * n_layers + 3 if fused_tail else 7 * n_layers + 4)
    g.replay()
    h_gpu = [t.to_numpy().copy() for t in trace]
    logits = gpu._graph_out[0].to_numpy().copy()
    tok = gpu._graph_out[1].to_numpy().copy()
    assert len(h_gpu) == cfg.num_hidden_layers + 1 and logits.shape == (B, cfg.vocab_size)
    np.testing.assert_array_equal(gpu.cache.seq_lens.to_numpy(), [ctx + 1] * B)
    np.testing.assert_array_equal(gpu._ids.numpy(), tok)
    np.testing.assert_array_equal(gpu._pos.numpy(), pos + 1)

    outs, tf_logits = cpu.decode_layers_teacher_forced(h_gpu, pos)
    for i in range(cfg.num_hidden_layers):
        err = float(np.abs(outs[i] - h_gpu[i + 1]).max())
        assert err <= 2e-3, (i, err)
        # the new token's cache row
        kc, vc = gpu.cache.get(i)
        gk, gv = kc.numpy()[:, :, ctx].astype(np.float32), vc.numpy()[:, :, ctx].astype(np.float32)
        wk, wv = cpu.k[i][:, :, ctx].astype(np.float32), cpu.v[i][:, :, ctx].astype(np.float32)
        # teacher-forced: every layer is a "layer 0" (identical input).  Of the 2048 activations entering the qkv
        # Linear a few flip by one fp16 ulp (up to 1.95e-3 for |x| in [2, 4)) times |w| up to 0.08: 3e-4 covers two
        # such flips in one output; a head's rms is about 0.9 at this width, so k carries the same term
        assert_cache_rows(gk, wk, 0, 3e-4)
        assert_cache_rows(gv, wv, 0, 3e-4)
        assert np.all(kc.numpy()[:, :, ctx + 1:] == 0)
    err = float(np.abs(tf_logits - logits).max())
    assert err <= 2e-3, err
    # the device's argmax over 151 936 columns is the argmax of the device's logits (first index on ties)
    np.testing.assert_array_equal(tok, logits.argmax(-1))
    chosen = tf_logits[np.arange(B), tok]
    assert np.all(chosen >= tf_logits.max(-1) - 4e-3)

    # second replay: the oracle steps from the first token on its own (its cache rows from the teacher-forced pass)
    g.replay()
    tok2 = gpu._graph_out[1].to_numpy().copy()
    c_logits, _ = cpu.decode_step(tok, pos + 1)
    chosen = c_logits[np.arange(B), tok2]
    assert np.all(chosen >= c_logits.max(-1) - 4e-3), (chosen, c_logits.max(-1))
    assert np.abs(gpu._graph_out[0].to_numpy() - c_logits).max() <= 2e-3 * n_layers   # free running: the per-layer bound adds up
    np.testing.assert_array_equal(gpu.cache.seq_lens.to_numpy(), [ctx + 2] * B)
    from axono_amd import libaxono as L
    assert L.decode_layer_tail_failed_waits() == 0
    print(f"real-width captured step: {time.perf_counter() - t_start:.1f} s")
