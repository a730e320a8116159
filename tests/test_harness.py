"""The Llama-architecture harness (llama_arch.py) that drives the operators the way the
reference's model.py does.  CPU: cache/position logic with torch restatements of the three
operators.  GPU: the same model with the HIP operators against the CPU run, at logits level
(greedy token streams of a random-init model are near ties and are not compared alone)."""

import numpy as np
import pytest
import torch

import llama_arch as la
from oracle import cpu_baseline


class CpuOps:
    rms_norm = staticmethod(cpu_baseline.rms_norm_cpu)
    rot_embed = staticmethod(cpu_baseline.rot_embed_cpu)
    flash_attention_decode = staticmethod(cpu_baseline.attention_cpu)


def tiny_config(**kw):
    base = dict(n_layer=2, vocab_size=1000, n_embd=256, n_head=4, n_kv_head=2, hidden_dim=512, max_model_len=48,
                max_gen_batch_size=3, block_size=64)
    base.update(kw)
    return la.LlamaConfig(**base)


def test_incremental_decode_matches_full_forward_cpu():
    """Prefill + single-token steps through the KV cache give the logits of one causal pass:
    pins the cache slice views, the start_pos rows of the rotary table and the T == 1 branch."""
    torch.manual_seed(0)
    cfg = tiny_config()
    m = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32)
    ids = torch.tensor(la.random_prompts(3, 12, 900, 5))
    with torch.inference_mode():
        inc = [m.forward(ids[:, :8], start_pos=0)]
        for p in range(8, 12):
            inc.append(m.forward(ids[:, p:p + 1], start_pos=p))
        for n, got in zip(range(8, 13), inc):
            full = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32).forward(ids[:, :n], start_pos=0)
            np.testing.assert_allclose(got.numpy(), full.numpy(), rtol=2e-4, atol=2e-5)


def test_generate_bookkeeping_cpu():
    cfg = tiny_config()
    m = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32)
    m.tokenizer.pad_id, m.tokenizer.stop_tokens = 999, (998,)
    prompts = [[5, 6, 7, 8], [9, 10]]        # ragged: the shorter row starts generating first
    out = m.generate(prompts, max_gen_len=5, ignore_eos=True)
    assert [len(o) for o in out] == [5, 5]
    echoed = m.generate(prompts, max_gen_len=5, echo=True, ignore_eos=True)
    assert echoed[0][:4] == prompts[0] and echoed[1][:2] == prompts[1]
    assert echoed[0][4:] == out[0][:len(echoed[0]) - 4]
    # greedy == argmax of the logits the forward pass returns
    with torch.inference_mode():
        m2 = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32)
        lg = m2.forward(torch.tensor([prompts[1]]), start_pos=0)
    assert out[1][0] == int(lg[0, -1].argmax())
    tps, dt, toks = la.timed_generate(m, 2, 6, 4)
    assert tps > 0 and len(toks) == 2 and all(len(t) == 4 for t in toks)
    with pytest.raises(NotImplementedError):
        m.generate(prompts, max_gen_len=2, temperature=0.6)


@pytest.mark.gpu
@pytest.mark.parametrize("n_kv_head,n_head", [(2, 4), (1, 4), (2, 16)])
def test_hip_operators_in_the_model_match_cpu_logits(gpu, n_kv_head, n_head):
    from custom_kernels import custom_kernels_extension as cke

    cfg = tiny_config(n_head=n_head, n_kv_head=n_kv_head, n_embd=64 * n_head)
    print(f"harness logits: heads {n_head}/{n_kv_head}", flush=True)
    ref = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32, seed=7)
    dut = la.LlamaDecoder(cfg, cke, gpu, dtype=torch.bfloat16, seed=7)
    # same weights: the reference model holds the bf16-rounded values in float32
    ref.wte = dut.wte.float().cpu()
    for Lr, Ld in zip(ref.layers, dut.layers):
        for key in ("c_attn", "c_proj", "c_fc", "c_fc2", "mlp_proj"):
            Lr[key] = Ld[key].float().cpu()
    ids = torch.tensor(la.random_prompts(3, 20, 900, 11))
    with torch.inference_mode():
        worst = 0.0
        for (lo, hi, sp) in [(0, 16, 0), (16, 17, 16), (17, 18, 17), (18, 19, 18), (19, 20, 19)]:
            a = ref.forward(ids[:, lo:hi], start_pos=sp)
            b = dut.forward(ids[:, lo:hi].to(gpu), start_pos=sp).cpu()
            scale = a.abs().max().item()
            err = (a - b).abs().max().item()
            worst = max(worst, err / scale)
            assert err <= 0.04 * scale, f"step at {sp}: logits differ by {err} (scale {scale})"
    print(f"  worst relative logit error {worst:.4f}", flush=True)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [5, 7, 12, 17, 20, 64])
def test_split_k_decode_path_matches_cpu_logits(gpu, rows):
    """5..64 sequences: the decode step goes through the split-K linears and the operators that add
    their splits up; logits against the float32 CPU model, step by step."""
    from custom_kernels import custom_kernels_extension as cke

    cfg = tiny_config(n_head=8, n_kv_head=2, n_embd=512, hidden_dim=1024, max_gen_batch_size=rows)
    ref = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32, seed=9)
    dut = la.LlamaDecoder(cfg, cke, gpu, dtype=torch.bfloat16, seed=9)
    assert dut._splitk(rows)
    ref.wte = dut.wte.float().cpu()
    for Lr, Ld in zip(ref.layers, dut.layers):
        for key in ("c_attn", "c_proj", "c_fc", "c_fc2", "mlp_proj"):
            Lr[key] = Ld[key].float().cpu()
    ids = torch.tensor(la.random_prompts(rows, 12, 900, 13))
    with torch.inference_mode():
        for (lo, hi, sp) in [(0, 9, 0), (9, 10, 9), (10, 11, 10), (11, 12, 11)]:
            print(f"split-k harness rows={rows} step at {sp}", flush=True)
            a = ref.forward(ids[:, lo:hi], start_pos=sp)
            b = dut.forward(ids[:, lo:hi].to(gpu), start_pos=sp).cpu()
            scale = a.abs().max().item()
            err = (a - b).abs().max().item()
            assert err <= 0.04 * scale, f"step at {sp}: logits differ by {err} (scale {scale})"


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 3, 4, 5, 9, 16, 20])
def test_graphed_decode_loop_matches_eager(gpu, batch):
    """The HIP-graph replay of the decode step against the eager loop, replay by replay: same
    logits path, same bookkeeping.  Checked over several generate() calls on one recorded graph
    (a graph that misbehaves from its second replay on would show here)."""
    from custom_kernels import custom_kernels_extension as cke

    cfg = tiny_config(n_head=8, n_kv_head=2, n_embd=512, max_gen_batch_size=max(4, batch), max_model_len=64)
    m = la.LlamaDecoder(cfg, cke, gpu, seed=3)
    m.tokenizer.pad_id, m.tokenizer.stop_tokens = 999, (998,)
    for seed in (1, 2, 3):
        prompts = la.random_prompts(batch, 9, 900, seed, exclude=())
        if batch > 1:
            prompts[1] = prompts[1][:5]           # ragged prompts: the mask-keep path
        print(f"graphed decode batch={batch} seed={seed}", flush=True)
        eager = m.generate(prompts, max_gen_len=20, ignore_eos=True)
        graphed = m.generate_graphed(prompts, max_gen_len=20, ignore_eos=True)
        torch.cuda.synchronize()
        # token streams of a random-init model can fork at a near-tie: require a long common prefix
        for a, b in zip(eager, graphed):
            common = 0
            for x, y in zip(a, b):
                if x != y:
                    break
                common += 1
            assert common >= 15, f"graphed and eager streams diverge after {common} tokens: {a} vs {b}"
    assert len(m._graphs) >= 1 and all(g.graph is not None for g in m._graphs.values())
    # the prompt pass of generate_graphed: whichever way it runs (recorded, or eager when the recording
    # failed its own check), new prompts through it give the eager pass's logits, replay after replay
    assert m.prefill_pass_mode() in ("recorded", "eager")
    print(f"prompt pass: {m.prefill_pass_mode()}", flush=True)
    assert all(len(loop.prefill_graphs) <= loop.MAX_PREFILL_GRAPHS for loop in m._graphs.values())
    with torch.inference_mode():
        for loop in m._graphs.values():
            for T in list(loop.prefill_graphs):
                for seed in (7, 8, 9):
                    g = torch.Generator().manual_seed(seed)
                    loop.tokens[:, :T] = torch.randint(0, 900, (loop.tokens.shape[0], T), generator=g).to(gpu)
                    got = loop.prefill(m, T).clone()
                    want = m.forward(loop.tokens[:, :T], start_pos=0)
                    assert torch.equal(got, want), f"prompt pass T={T} seed={seed}"


@pytest.mark.gpu
def test_only_the_last_few_prompt_lengths_stay_recorded(gpu):
    """Six prompt lengths on one decode loop (same batch, same total length): every generation matches the
    eager one, and the loop holds no more recorded prompt passes than its limit."""
    from custom_kernels import custom_kernels_extension as cke

    cfg = tiny_config(n_head=8, n_kv_head=2, n_embd=512, max_gen_batch_size=2, max_model_len=64)
    m = la.LlamaDecoder(cfg, cke, gpu, seed=6)
    m.tokenizer.pad_id, m.tokenizer.stop_tokens = 999, (998,)
    for n in range(5, 11):
        prompts = la.random_prompts(1, n, 900, n, exclude=())
        print(f"prompt length {n}", flush=True)
        eager = m.generate(prompts, max_gen_len=30 - n, ignore_eos=True)
        graphed = m.generate_graphed(prompts, max_gen_len=30 - n, ignore_eos=True)
        torch.cuda.synchronize()
        assert eager[0][:8] == graphed[0][:8], f"streams diverge early: {eager[0]} vs {graphed[0]}"
    assert len(m._graphs) == 1
    loop = next(iter(m._graphs.values()))
    assert len(loop.prefill_graphs) == loop.MAX_PREFILL_GRAPHS and 10 in loop.prefill_graphs and 5 not in loop.prefill_graphs


@pytest.mark.gpu
def test_prompt_pass_falls_back_to_eager_when_its_recording_fails_the_check(gpu, monkeypatch):
    """A recorded prompt pass that does not reproduce the eager logits must not be used: with the
    comparison forced to fail, generate_graphed keeps the eager pass and still matches generate()."""
    from custom_kernels import custom_kernels_extension as cke

    cfg = tiny_config(n_head=8, n_kv_head=2, n_embd=512, max_gen_batch_size=4, max_model_len=64)
    m = la.LlamaDecoder(cfg, cke, gpu, seed=5)
    m.tokenizer.pad_id, m.tokenizer.stop_tokens = 999, (998,)
    prompts = la.random_prompts(2, 9, 900, 4, exclude=())
    eager = m.generate(prompts, max_gen_len=12, ignore_eos=True)
    monkeypatch.setattr(torch, "equal", lambda a, b: False)
    graphed = m.generate_graphed(prompts, max_gen_len=12, ignore_eos=True)
    torch.cuda.synchronize()
    monkeypatch.undo()
    assert m.prefill_pass_mode() == "eager"
    for a, b in zip(eager, graphed):
        assert a[:8] == b[:8], f"streams diverge early: {a} vs {b}"


# ---- the end-to-end configuration at its own size (Llama-3.2-1B architecture, model.py:153-166;
#      benchmark_model.py:69-85 drives it with 128 prompt ids and 128 generated tokens)
@pytest.fixture(scope="module")
def full_size_model(gpu):
    from custom_kernels import custom_kernels_extension as cke

    cfg = la.LlamaConfig(max_model_len=256, max_gen_batch_size=64)
    assert (cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.n_kv_head, cfg.hidden_dim, cfg.vocab_size) == \
        (16, 2048, 32, 8, 8192, 128256)
    print("full-size harness: building the 1B-shaped model", flush=True)
    m = la.LlamaDecoder(cfg, cke, gpu, seed=5)
    yield m
    del m
    torch.cuda.empty_cache()


@pytest.mark.gpu
def test_full_size_logits_match_cpu_model(gpu, full_size_model):
    """Prefill of 128 tokens and the first two decode steps at batch 2: logits against the float32
    CPU model holding the same bf16-rounded weights, within 4 % of the logit range."""
    dut = full_size_model
    cfg = la.LlamaConfig(max_model_len=256, max_gen_batch_size=2)
    ref = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32, weights_from=dut)
    ids = torch.tensor(la.random_prompts(2, 130, cfg.vocab_size, 21))
    with torch.inference_mode():
        for (lo, hi, sp) in [(0, 128, 0), (128, 129, 128), (129, 130, 129)]:
            print(f"full-size logits: tokens {lo}..{hi} at {sp}", flush=True)
            a = ref.forward(ids[:, lo:hi], start_pos=sp)
            b = dut.forward(ids[:, lo:hi].to(gpu), start_pos=sp).cpu()
            scale = a.abs().max().item()
            err = (a - b).abs().max().item()
            assert err <= 0.04 * scale, f"step at {sp}: logits differ by {err} (scale {scale})"
    del ref


@pytest.mark.gpu
def test_full_size_logits_match_cpu_model_on_the_split_k_route(gpu, full_size_model):
    """Batch 5 is the first batch size whose output and down projections take the split-K kernels (float32
    partial products summed by the operator that follows) and whose qkv / gate|up linears run with more than
    four activation rows: a 16-token prompt and two decode steps at the 1B shape against the float32 CPU
    model, within 4 % of the logit range."""
    dut = full_size_model
    assert la.LlamaDecoder.FUSED_MAX_ROWS < 5 <= la.LlamaDecoder.QKV_FUSED_MAX_ROWS
    cfg = la.LlamaConfig(max_model_len=256, max_gen_batch_size=5)
    ref = la.LlamaDecoder(cfg, CpuOps, "cpu", dtype=torch.float32, weights_from=dut)
    ids = torch.tensor(la.random_prompts(5, 18, cfg.vocab_size, 23))
    with torch.inference_mode():
        for (lo, hi, sp) in [(0, 16, 0), (16, 17, 16), (17, 18, 17)]:
            print(f"full-size logits, batch 5: tokens {lo}..{hi} at {sp}", flush=True)
            a = ref.forward(ids[:, lo:hi], start_pos=sp)
            b = dut.forward(ids[:, lo:hi].to(gpu), start_pos=sp).cpu()
            scale = a.abs().max().item()
            err = (a - b).abs().max().item()
            assert err <= 0.04 * scale, f"step at {sp}: logits differ by {err} (scale {scale})"
    del ref


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 64])
def test_full_size_graphed_loop_matches_eager(gpu, full_size_model, batch):
    """128 prompt ids + 128 greedy tokens at batch 1 (fused single-launch linears) and batch 64
    (library GEMMs, strided gate|up halves): the HIP-graph replay against the eager loop.  The two
    loops plan the attention splits differently (device-side against host-side KV length), so a
    near-tie may fork a stream: a long common prefix and broad agreement are required, not identity."""
    m = full_size_model
    prompts = la.random_prompts(batch, 128, m.config.vocab_size, 31)
    print(f"full-size generate: batch {batch}", flush=True)
    eager = m.generate(prompts, max_gen_len=128, ignore_eos=True)
    graphed = m.generate_graphed(prompts, max_gen_len=128, ignore_eos=True)
    torch.cuda.synchronize()
    agree = total = 0
    for a, b in zip(eager, graphed):
        assert len(a) == len(b) == 128
        common = 0
        for x, y in zip(a, b):
            if x != y:
                break
            common += 1
        assert common >= 100, f"graphed and eager streams diverge after {common} tokens"
        agree += common
        total += len(a)
    assert agree >= 0.98 * total, f"only {agree} of {total} tokens lie in common prefixes"
