"""End-to-end: random-init models through `optimize_model` on the GPU against the fp32 eager model on the CPU.

Follows the reference's test/test_model_optimization.py:25-41 and test/test_torchdynamo.py:60-100 (BERT over several
shapes, shape change without rebuilding).  Pretrained checkpoints are not reachable offline; the models are built from
their config classes with seed 0, as BASELINE configs 0 and 3 prescribe.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _bert(layers=12, attn="eager"):
    from transformers import BertConfig, BertModel

    torch.manual_seed(0)
    cfg = BertConfig(num_hidden_layers=layers)
    cfg._attn_implementation = attn
    return BertModel(cfg).eval()


def _inputs(batch, seq, gen, min_len=None):
    ids = torch.randint(0, 30522, (batch, seq), generator=gen)
    lengths = torch.randint(min_len or max(1, seq // 2), seq + 1, (batch,), generator=gen)
    mask = (torch.arange(seq)[None, :] < lengths[:, None]).long()
    return ids, mask


def _compare(out, ref, mask, what):
    a, e = out.float().cpu(), ref.float()
    assert torch.isfinite(a).all(), what
    valid = mask.bool()
    diff = (a - e).abs()
    # tolerance stated by BASELINE for fp16 hidden states: max-abs <= 1e-2 x scale, mean-rel <= 1e-3 x 10 after 12 layers
    max_abs = diff[valid].max().item()
    mean_rel = (diff[valid].mean() / e[valid].abs().mean()).item()
    print(f"{what}: max_abs={max_abs:.4f} mean_rel={mean_rel:.5f}", flush=True)
    assert max_abs <= 5e-2, f"{what}: max abs error {max_abs}"
    assert mean_rel <= 5e-3, f"{what}: mean relative error {mean_rel}"


@pytest.mark.parametrize("attn", ["eager", "sdpa"])
def test_bert_base_matches_fp32_eager(attn):
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(0)
    ref_model = _bert(attn=attn)
    ids, mask = _inputs(4, 128, gen)
    with torch.inference_mode():
        ref = ref_model(input_ids=ids, attention_mask=mask).last_hidden_state
    model = _bert(attn=attn).half().cuda()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state
        torch.cuda.synchronize()
        _compare(out, ref, mask, f"bert-base {attn} (4,128)")
        # replay with different values at the same shape
        ids2, mask2 = _inputs(4, 128, gen)
        ref2 = ref_model(input_ids=ids2, attention_mask=mask2).last_hidden_state
        out2 = model(input_ids=ids2.cuda(), attention_mask=mask2.cuda()).last_hidden_state
        torch.cuda.synchronize()
        _compare(out2, ref2, mask2, f"bert-base {attn} replay")


@pytest.mark.parametrize("batch, seq", [(1, 16), (1, 128), (1, 512), (8, 128)], ids=lambda v: str(v))
def test_bert_base_over_the_reference_shape_grid(batch, seq):
    """The 12-layer model at shapes of the reference's grid (test/test_torchdynamo.py:38-57 runs batch 1, 8, 32 x
    16 .. 512 tokens): batch 1 puts 12 heads on 256 CUs (the small-grid attention and few-row linear routes), 16 tokens
    is less than one key tile, and every shape is captured and replayed as a graph of its own."""
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(batch * 1000 + seq)
    ref_model = _bert()
    model = _bert().half().cuda()
    optimize_model(model)
    for rep in range(2):  # the second pass replays the captured graph on other values
        ids, mask = _inputs(batch, seq, gen)
        with torch.inference_mode():
            ref = ref_model(input_ids=ids, attention_mask=mask).last_hidden_state
            out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state
            torch.cuda.synchronize()
        _compare(out, ref, mask, f"bert-base ({batch},{seq}) pass {rep}")


def test_bert_base_config3_full_size():
    """BASELINE config 3 at its stated size: BERT-base (seed 0) in fp16 through `optimize_model`, forward captured in a
    hipGraph, batch 32 x 512 tokens, lengths U[256, 512] — final hidden states against the fp32 eager model on the
    CPU (counterpart of the reference's test/test_torchdynamo.py:60-83, which stops at 1e-1).  The full-size shapes
    take kernel paths the smaller cases do not: more GEMM tiles than CUs in the persistent kernel, the 256x192 tile
    choice, fused add + LayerNorm over 16384 rows, 1536 attention workgroups."""
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(0)
    ids, mask = _inputs(32, 512, gen, min_len=256)
    ref_model = _bert()
    with torch.inference_mode():
        ref = ref_model(input_ids=ids, attention_mask=mask).last_hidden_state
    model = _bert().half().cuda()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state  # warm-up + capture
        out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state  # replay
        torch.cuda.synchronize()
    _compare(out, ref, mask, "bert-base config 3 (32,512)")
    # padded query rows are deterministic too (they attend to the valid keys): the whole tensor is finite and close
    diff_all = (out.float().cpu() - ref).abs()
    assert diff_all.max().item() <= 1e-1, diff_all.max().item()


def test_bert_shape_change_without_rebuild():
    # reference test/test_torchdynamo.py:86-100
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(1)
    ref_model = _bert(layers=2)
    model = _bert(layers=2).half().cuda()
    optimize_model(model)
    for shape in [(1, 64), (8, 256), (16, 256), (16, 64), (1, 64)]:
        ids, mask = _inputs(*shape, gen)
        with torch.inference_mode():
            ref = ref_model(input_ids=ids, attention_mask=mask).last_hidden_state
            out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state
            torch.cuda.synchronize()
        _compare(out, ref, mask, f"bert 2 layers {shape}")


def test_autocast_fp32_model():
    # reference test/test_model_optimization.py:25-41: fp32 weights, fp16 autocast
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(2)
    ref_model = _bert(layers=2)
    model = _bert(layers=2).cuda()
    optimize_model(model)
    ids, mask = _inputs(1, 128, gen)
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.float16):
        out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state
        out = model(input_ids=ids.cuda(), attention_mask=mask.cuda()).last_hidden_state
        torch.cuda.synchronize()
    with torch.inference_mode():
        ref = ref_model(input_ids=ids, attention_mask=mask).last_hidden_state
    _compare(out, ref, mask, "bert autocast")


def _llama(layers, hidden, heads, inter, attn="sdpa", vocab=1000, eps=1e-5):
    from transformers import LlamaConfig, LlamaModel

    torch.manual_seed(0)
    cfg = LlamaConfig(num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=heads,
                      intermediate_size=inter, vocab_size=vocab, rms_norm_eps=eps, max_position_embeddings=4096)
    cfg._attn_implementation = attn
    return LlamaModel(cfg).eval()


@pytest.mark.parametrize("attn", ["eager", "sdpa"])
def test_llama_shaped_decoder_matches_fp32_eager(attn):
    # BASELINE config 4 in miniature: causal prefill, head size 128, RoPE, SwiGLU, RMSNorm eps 1e-5
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 1000, (2, 320), generator=gen)
    # The fp32 reference keeps the config's eps (1e-5).  The fp16 operator clamps eps to >= 1.6e-5 (reference
    # layer_norm.py:295-296, applied to RMSNorm as well); with N(0, 0.02) weights the hidden states have variance
    # ~4e-4, where that moves rstd by 0.7 %.  What the clamp alone does to the output is measured on the fp32 model
    # (same weights, eps 1.6e-5) and added to the bound.
    ref_model = _llama(2, 512, 4, 1408, attn)
    with torch.inference_mode():
        ref = ref_model(input_ids=ids, use_cache=False).last_hidden_state
        ref_clamped = _llama(2, 512, 4, 1408, attn, eps=1.6e-5)(input_ids=ids, use_cache=False).last_hidden_state
    clamp_rel = ((ref_clamped - ref).abs().mean() / ref.abs().mean()).item()
    model = _llama(2, 512, 4, 1408, attn).half().cuda()
    with torch.inference_mode():
        eager16 = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state.float().cpu()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        torch.cuda.synchronize()
    # plain fp16 eager (eps 1e-5, unclamped) is printed beside ours for orientation
    eager_rel = ((eager16 - ref).abs().mean() / ref.abs().mean()).item()
    ours_rel = ((out.float().cpu() - ref).abs().mean() / ref.abs().mean()).item()
    print(f"llama-shaped {attn}: mean_rel ours={ours_rel:.5f} fp16-eager={eager_rel:.5f} eps-clamp alone={clamp_rel:.5f}", flush=True)
    assert torch.isfinite(out).all()
    assert ours_rel <= 5e-3 + clamp_rel
    assert (out.float().cpu() - ref).abs().max().item() <= 1e-1


def test_llama_shaped_short_input_runs_the_one_launch_norm_projections(monkeypatch):
    """24 tokens (at most 64 rows): both RMSNorms of every layer run inside the projections they feed — the fused
    query/key/value projection together with the rotation of queries and keys (`kernl_linear_decode_fwd`), the gated
    feed-forward entry (`kernl_linear_rms_fwd`) — and the result still matches the fp32 model.  (The output and down
    projections of a model this narrow are shapes of the one-launch small-tile kernels, which beat the weight-streaming
    kernel by more than a separate addition costs: no residual rides in a projection here.)"""
    from kernl_amd import _lib
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    calls = {"rms": 0, "gated": 0, "rotating": 0, "residual": 0}
    real = _lib.linear_rms_fwd
    real_decode = _lib.linear_decode_fwd

    def counting(x2d, rms_weight, eps, weight, bias, out2d, activation, gated):
        calls["rms"] += 1
        calls["gated"] += int(bool(gated))
        return real(x2d, rms_weight, eps, weight, bias, out2d, activation, gated)

    def counting_decode(x2d, rms_weight, eps, weight, bias, residual2d, out2d, cos=None, sin=None, *args, **kwargs):
        calls["rotating"] += int(cos is not None and rms_weight is not None)
        calls["residual"] += int(residual2d is not None)
        return real_decode(x2d, rms_weight, eps, weight, bias, residual2d, out2d, cos, sin, *args, **kwargs)

    monkeypatch.setattr(_lib, "linear_decode_fwd", counting_decode)
    monkeypatch.setattr(_lib, "linear_rms_fwd", counting)
    gen = torch.Generator().manual_seed(6)
    ids = torch.randint(0, 1000, (2, 12), generator=gen)
    ref_model = _llama(2, 512, 4, 1408, "sdpa")
    with torch.inference_mode():
        ref = ref_model(input_ids=ids, use_cache=False).last_hidden_state
        ref_clamped = _llama(2, 512, 4, 1408, "sdpa", eps=1.6e-5)(input_ids=ids, use_cache=False).last_hidden_state
    clamp_rel = ((ref_clamped - ref).abs().mean() / ref.abs().mean()).item()  # what the operator's fp16 eps clamp alone does
    model = _llama(2, 512, 4, 1408, "sdpa").half().cuda()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        torch.cuda.synchronize()
    # warm-up and capture each run the two layers once: 2 x 2 x (one rotating q/k/v projection, one gated feed-forward entry)
    assert calls == {"rms": 4, "gated": 4, "rotating": 4, "residual": 0}, calls
    ours_rel = ((out.float().cpu() - ref).abs().mean() / ref.abs().mean()).item()
    print(f"llama-shaped, 24 rows: mean_rel ours={ours_rel:.5f}", flush=True)
    assert torch.isfinite(out).all() and ours_rel <= 5e-3 + clamp_rel


def test_llama_7b_shaped_layer_full_width():
    # one decoder layer at Llama-2-7B width (4096, 32 heads of 128, SwiGLU 11008), batch 1, 2048 tokens, causal.
    # With N(0, 0.02) random weights attention is close to uniform over up to 2048 keys and fp16 itself is several
    # per cent away from fp32 at late positions (plain fp16 eager PyTorch: ~5 %, growing with the position), so the
    # bar here is "no further from the fp32 model than fp16 eager PyTorch is", plus exact agreement of the pieces in
    # the kernel-level tests.
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(4)
    ids = torch.randint(0, 1000, (1, 2048), generator=gen)
    ref_model = _llama(1, 4096, 32, 11008)  # the config's own eps (1e-5)
    with torch.inference_mode():
        ref = ref_model(input_ids=ids, use_cache=False).last_hidden_state
        # what the operator's fp16 eps clamp (>= 1.6e-5, reference layer_norm.py:295-296) alone does, on the fp32 model
        ref_clamped = _llama(1, 4096, 32, 11008, eps=1.6e-5)(input_ids=ids, use_cache=False).last_hidden_state
    clamp_rel = ((ref_clamped - ref).abs().mean() / ref.abs().mean()).item()
    model = _llama(1, 4096, 32, 11008).half().cuda()
    with torch.inference_mode():
        eager16 = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state.float().cpu()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        torch.cuda.synchronize()
    eager_rel = ((eager16 - ref).abs().mean() / ref.abs().mean()).item()
    ours_rel = ((out.float().cpu() - ref).abs().mean() / ref.abs().mean()).item()
    early = ((out.float().cpu() - ref)[:, :64].abs().mean() / ref[:, :64].abs().mean()).item()
    print(f"llama-7b-shaped layer: mean_rel ours={ours_rel:.5f} fp16-eager={eager_rel:.5f} eps-clamp alone={clamp_rel:.5f} "
          f"ours(first 64 positions)={early:.5f}", flush=True)
    assert torch.isfinite(out).all()
    assert ours_rel <= max(5e-3, 1.1 * eager_rel) + clamp_rel
    assert early <= 5e-3 + clamp_rel


def _rel_errors(out, eager16, ref):
    ours = ((out.float().cpu() - ref).abs().mean() / ref.abs().mean()).item()
    eager = ((eager16 - ref).abs().mean() / ref.abs().mean()).item()
    return ours, eager


def test_llama_7b_shaped_four_layers_full_width():
    """BASELINE config 4 at full width and length, four of its 32 layers: hidden 4096, 32 heads of 128, SwiGLU 11008,
    RoPE base 10000, RMSNorm eps 1e-5, weights N(0, 0.02), batch 1 x 2048 tokens, causal prefill through
    `optimize_model` — against the fp32 eager model on the CPU, which keeps the config's eps.  The fp16 operator clamps
    eps to >= 1.6e-5 (reference layer_norm.py:295-296); what that alone does is measured on the fp32 model and added to
    the bound, and plain fp16 eager PyTorch is printed beside ours.  With random weights attention is close to
    uniform over up to 2048 keys and fp16 accumulates error with depth and position, so the bound is "no further from
    fp32 than fp16 eager PyTorch" with 10 % slack, and 5e-3 on the first 64 positions."""
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    gen = torch.Generator().manual_seed(7)
    ids = torch.randint(0, 1000, (1, 2048), generator=gen)
    with torch.inference_mode():
        ref = _llama(4, 4096, 32, 11008)(input_ids=ids, use_cache=False).last_hidden_state
        ref_clamped = _llama(4, 4096, 32, 11008, eps=1.6e-5)(input_ids=ids, use_cache=False).last_hidden_state
    clamp_rel = ((ref_clamped - ref).abs().mean() / ref.abs().mean()).item()
    del ref_clamped
    model = _llama(4, 4096, 32, 11008).half().cuda()
    with torch.inference_mode():
        eager16 = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state.float().cpu()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        out = model(input_ids=ids.cuda(), use_cache=False).last_hidden_state
        torch.cuda.synchronize()
    ours, eager = _rel_errors(out, eager16, ref)
    early = ((out.float().cpu() - ref)[:, :64].abs().mean() / ref[:, :64].abs().mean()).item()
    print(f"llama-7b-shaped, 4 layers: mean_rel ours={ours:.5f} fp16-eager={eager:.5f} eps-clamp alone={clamp_rel:.5f} "
          f"ours(first 64 positions)={early:.5f}", flush=True)
    assert torch.isfinite(out).all()
    assert ours <= max(5e-3, 1.1 * eager) + clamp_rel
    assert early <= 5e-3 + clamp_rel


def test_llama_7b_shaped_at_its_full_depth():
    """BASELINE config 4 as stated: 32 layers at full width, batch 1 x 2048 tokens (13.5 GB of fp16 weights created on the
    GPU), causal prefill through `optimize_model` — the run `bench.py` times.  The reference values are the SAME weights
    in fp32 on the GPU with the operators' fp16 eps clamp (reference layer_norm.py:295-296) built in, so that what is left
    is the fp16 arithmetic: ours must be no further from them than eager fp16 PyTorch is, with 25 % slack (both sit near
    1 % after 32 layers of N(0, 0.02) weights)."""
    import bench

    if torch.cuda.get_device_properties(0).total_memory < 80e9:
        pytest.skip("needs 60 GB of device memory")
    r = bench.llama7b_prefill(torch.device("cuda:0"))
    ours = r["llama7b_b1_s2048_mean_rel_err_vs_fp32_model_with_clamped_eps"]
    eager = r["llama7b_b1_s2048_fp16_eager_mean_rel_err_vs_fp32_model_with_clamped_eps"]
    print(f"llama-7b-shaped, 32 layers: mean_rel vs fp32 ours={ours:.5f} fp16-eager={eager:.5f}, "
          f"{r['llama7b_b1_s2048_fwd_ms']} ms per forward", flush=True)
    assert ours <= 1.25 * eager + 1e-3
    torch._dynamo.reset()


@pytest.mark.parametrize("attn", ["eager", "sdpa"])
def test_t5_shaped_encoder_decoder_matches_fp32_eager(attn):
    """T5 (reference: test/test_torchdynamo.py:102-131, t5-small): relative position bias as a matrix mask in encoder
    and decoder self-attention, cross-attention without a mask, T5-spelled RMSNorm, ReLU feed-forward.  Random-init
    t5-small-shaped model, two layers, encoder 128 tokens, decoder 48."""
    from transformers import T5Config, T5Model

    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()

    def make():
        torch.manual_seed(0)
        cfg = T5Config(d_model=512, d_kv=64, d_ff=2048, num_layers=2, num_heads=8, vocab_size=1000,
                       layer_norm_epsilon=1.6e-5)  # the fp16 operator clamps eps to >= 1.6e-5 (layer_norm.py:295-296)
        cfg._attn_implementation = attn
        return T5Model(cfg).eval()

    gen = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 1000, (4, 128), generator=gen)
    dec = torch.randint(0, 1000, (4, 48), generator=gen)
    with torch.inference_mode():
        ref = make()(input_ids=ids, decoder_input_ids=dec, use_cache=False).last_hidden_state
    model = make().half().cuda()
    with torch.inference_mode():
        eager16 = model(input_ids=ids.cuda(), decoder_input_ids=dec.cuda(), use_cache=False).last_hidden_state.float().cpu()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_ids=ids.cuda(), decoder_input_ids=dec.cuda(), use_cache=False).last_hidden_state
        out = model(input_ids=ids.cuda(), decoder_input_ids=dec.cuda(), use_cache=False).last_hidden_state
        torch.cuda.synchronize()
    ours, eager = _rel_errors(out, eager16, ref)
    print(f"t5-shaped {attn}: mean_rel ours={ours:.5f} fp16-eager={eager:.5f}", flush=True)
    assert torch.isfinite(out).all()
    assert ours <= 5e-3
    assert (out.float().cpu() - ref).abs().max().item() <= 1e-1 * max(1.0, ref.abs().max().item())


@pytest.mark.parametrize("attn", ["eager", "sdpa"])
def test_whisper_shaped_encoder_decoder_matches_fp32_eager(attn):
    """Whisper (reference: test/test_torchdynamo.py:134-165, whisper-tiny): 1500 encoder positions (not a multiple of
    any tile), bmm-shaped attention without a mask in the encoder, causal decoder self-attention, cross-attention,
    LayerNorm with residual adds, GELU feed-forward.  Random-init whisper-tiny-shaped model with two layers."""
    from transformers import WhisperConfig, WhisperModel

    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()

    def make():
        torch.manual_seed(0)
        cfg = WhisperConfig(d_model=384, encoder_layers=2, decoder_layers=2, encoder_attention_heads=6,
                            decoder_attention_heads=6, encoder_ffn_dim=1536, decoder_ffn_dim=1536, vocab_size=1000,
                            pad_token_id=0, bos_token_id=1, eos_token_id=2, decoder_start_token_id=1, num_mel_bins=80,
                            max_source_positions=1500, max_target_positions=64)
        cfg._attn_implementation = attn
        return WhisperModel(cfg).eval()

    gen = torch.Generator().manual_seed(6)
    feats = torch.randn((2, 80, 3000), generator=gen)
    dec = torch.randint(3, 1000, (2, 24), generator=gen)
    with torch.inference_mode():
        ref = make()(input_features=feats, decoder_input_ids=dec, use_cache=False).last_hidden_state
    model = make().half().cuda()
    with torch.inference_mode():
        eager16 = model(input_features=feats.half().cuda(), decoder_input_ids=dec.cuda(), use_cache=False).last_hidden_state.float().cpu()
    optimize_model(model)
    with torch.inference_mode():
        out = model(input_features=feats.half().cuda(), decoder_input_ids=dec.cuda(), use_cache=False).last_hidden_state
        out = model(input_features=feats.half().cuda(), decoder_input_ids=dec.cuda(), use_cache=False).last_hidden_state
        torch.cuda.synchronize()
    ours, eager = _rel_errors(out, eager16, ref)
    print(f"whisper-shaped {attn}: mean_rel ours={ours:.5f} fp16-eager={eager:.5f}", flush=True)
    assert torch.isfinite(out).all()
    assert ours <= 5e-3
    assert (out.float().cpu() - ref).abs().max().item() <= 1e-1 * max(1.0, ref.abs().max().item())


@pytest.mark.parametrize("family", ["t5", "whisper"])
def test_generation_with_growing_cache(family):
    """Greedy generation under autocast with `optimize_model` on encoder and decoder, as the reference tests it
    (test/test_torchdynamo.py:102-165): every decoding step meets a longer key/value cache, i.e. a new shape, a new
    compilation and a new captured graph; single-query attention runs on the split-K kernel.  Checks that no step falls
    back to the unoptimised function (TorchDynamo's recompile limit) and that the per-step scores follow the eager
    model's for as long as the two greedy paths pick the same tokens."""
    from torch._dynamo.utils import counters

    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    counters.clear()
    torch.manual_seed(0)
    gen = torch.Generator().manual_seed(1)
    if family == "t5":
        from transformers import T5Config, T5ForConditionalGeneration

        cfg = T5Config(d_model=512, d_kv=64, d_ff=2048, num_layers=2, num_heads=8, vocab_size=1000,
                       decoder_start_token_id=0, pad_token_id=0, eos_token_id=1, tie_word_embeddings=False)
        model = T5ForConditionalGeneration(cfg).eval().cuda()
        ids = torch.randint(2, 1000, (2, 64), generator=gen).cuda()
        kwargs = dict(input_ids=ids, attention_mask=torch.ones_like(ids))
        encoder, decoder = model.encoder, model.decoder
    else:
        from transformers import WhisperConfig, WhisperForConditionalGeneration

        cfg = WhisperConfig(d_model=384, encoder_layers=2, decoder_layers=2, encoder_attention_heads=6,
                            decoder_attention_heads=6, encoder_ffn_dim=1536, decoder_ffn_dim=1536, vocab_size=1000,
                            pad_token_id=0, bos_token_id=1, eos_token_id=2, decoder_start_token_id=1, num_mel_bins=80,
                            max_source_positions=1500, max_target_positions=64, suppress_tokens=None,
                            begin_suppress_tokens=None)
        model = WhisperForConditionalGeneration(cfg).eval().cuda()
        model.generation_config.suppress_tokens = None
        model.generation_config.begin_suppress_tokens = None
        model.generation_config.forced_decoder_ids = None
        kwargs = dict(input_features=torch.randn((2, 80, 3000), generator=gen).cuda())
        encoder, decoder = model.model.encoder, model.model.decoder
    steps = 20
    kwargs.update(min_new_tokens=steps, max_new_tokens=steps, do_sample=False, output_scores=True, return_dict_in_generate=True)
    with torch.inference_mode(), torch.autocast(dtype=torch.float16, device_type="cuda"):
        ref = model.generate(**kwargs)
    optimize_model(encoder)
    optimize_model(decoder)
    with torch.inference_mode(), torch.autocast(dtype=torch.float16, device_type="cuda"):
        model.generate(**kwargs)        # compiles and captures one graph per step
        out = model.generate(**kwargs)  # replays them
        torch.cuda.synchronize()
    frames = counters["frames"]
    assert frames["ok"] == frames["total"], f"some steps were not compiled: {dict(frames)}"
    assert counters["stats"]["unique_graphs"] >= steps, dict(counters["stats"])
    assert len(out.scores) == len(ref.scores) == steps
    prompt = ref.sequences.shape[1] - steps
    agree = 0
    for t, (a, b) in enumerate(zip(out.scores, ref.scores)):
        if not torch.equal(out.sequences[:, : prompt + t], ref.sequences[:, : prompt + t]):
            break
        finite = torch.isfinite(b)
        assert torch.equal(torch.isfinite(a), finite)
        scale = b[finite].abs().max().item()
        diff = (a.float() - b.float())[finite].abs().max().item()
        assert diff <= 4e-3 * max(scale, 1.0), f"{family} step {t}: scores differ by {diff} (scale {scale})"
        agree += 1
    print(f"{family}: greedy paths agree for {agree} of {steps} steps", flush=True)
    assert agree >= 3


@pytest.mark.parametrize("batch, hidden, heads, inter", [(2, 512, 4, 1408), (24, 2048, 16, 5632)], ids=["b2-h512", "b24-h2048"])
def test_llama_generation_runs_the_decode_projection_kernel(batch, hidden, heads, inter, monkeypatch):
    """Greedy generation with a growing key/value cache on a Llama-shaped fp16 model under `optimize_model`: each
    decoding step is a new cache length, hence a new compilation and graph.  In the steps after the prompt every layer's
    query/key/value projection must run as one call of the few-row projection kernel with the RMS prologue and the
    rotation, and the output and down projections as calls with the residual; the scores follow the eager fp16
    model's while the two greedy paths pick the same tokens.  With 24 sequences and 2048-wide layers the decoding steps
    have enough rows and weights for the stream-K form of those kernels (and of the gated feed-forward entry)."""
    from torch._dynamo.utils import counters
    from transformers import LlamaConfig, LlamaForCausalLM

    from kernl_amd import _lib
    from kernl_amd.model_optimization import optimize_model

    torch._dynamo.reset()
    counters.clear()
    torch.manual_seed(0)
    layers, steps = 2, 12
    cfg = LlamaConfig(num_hidden_layers=layers, hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=heads,
                      intermediate_size=inter, vocab_size=1000, rms_norm_eps=1e-5, max_position_embeddings=512,
                      pad_token_id=0, bos_token_id=1, eos_token_id=2)
    cfg._attn_implementation = "sdpa"
    model = LlamaForCausalLM(cfg).eval().half().cuda()
    gen = torch.Generator().manual_seed(1)
    ids = torch.randint(3, 1000, (batch, 20), generator=gen).cuda()
    kwargs = dict(input_ids=ids, attention_mask=torch.ones_like(ids), min_new_tokens=steps, max_new_tokens=steps,
                  do_sample=False, output_scores=True, return_dict_in_generate=True)
    # The model under test keeps the config's eps (1e-5).  The fp16 RMSNorm operator clamps eps to 1.6e-5 (reference
    # layer_norm.py:295-296): with N(0, 0.02) weights that alone moves the first step's scores by about 1 % of their
    # range, printed below.  The per-step bound is therefore taken against the eager model run with the clamped eps.
    norms = [m for m in model.modules() if type(m).__name__ == "LlamaRMSNorm"]
    with torch.inference_mode():
        config_eps = model.generate(**kwargs)
        for m in norms:
            m.variance_epsilon = 1.6e-5
        ref = model.generate(**kwargs)
        for m in norms:
            m.variance_epsilon = 1e-5
    first = torch.isfinite(ref.scores[0])
    clamp_effect = (ref.scores[0].float() - config_eps.scores[0].float())[first].abs().max().item()
    print(f"eps clamp alone moves the first scores by {clamp_effect:.4f} (range {ref.scores[0][first].abs().max().item():.2f})", flush=True)

    calls = {"rotated": 0, "residual": 0, "gated": 0}
    real, real_few = _lib.linear_decode_fwd, _lib.linear_fewrow_fwd

    def counting(x2d, rms_weight, eps, weight, bias, residual2d, out2d, cos=None, sin=None, *args, **kw):
        assert batch == 2, "24 rows belong on the stream-K kernel"
        calls["rotated"] += int(cos is not None and rms_weight is not None)
        calls["residual"] += int(residual2d is not None)
        return real(x2d, rms_weight, eps, weight, bias, residual2d, out2d, cos, sin, *args, **kw)

    def counting_few(x2d, weight, bias, residual2d, out2d, activation, workspace=None, **kw):
        assert batch == 24 and x2d.shape[0] == batch
        calls["rotated"] += int(kw.get("cos") is not None and kw.get("rms_weight") is not None)
        calls["residual"] += int(residual2d is not None)
        calls["gated"] += int(bool(kw.get("gated")) and kw.get("rms_weight") is not None)
        return real_few(x2d, weight, bias, residual2d, out2d, activation, workspace, **kw)

    monkeypatch.setattr(_lib, "linear_decode_fwd", counting)
    monkeypatch.setattr(_lib, "linear_fewrow_fwd", counting_few)
    optimize_model(model.model)
    with torch.inference_mode():
        model.generate(**kwargs)        # compiles and captures one graph per step
        out = model.generate(**kwargs)  # replays them
        torch.cuda.synchronize()
    frames = counters["frames"]
    assert frames["ok"] == frames["total"], f"some steps were not compiled: {dict(frames)}"
    assert counters["stats"]["unique_graphs"] >= steps, dict(counters["stats"])
    # warm-up run and capture run of each of the steps after the prompt
    assert calls["rotated"] >= 2 * (steps - 1) * layers, calls
    # (24 rows against the 2048 x 2048 output projection is a shape of the one-launch small-tile kernels, which keep the
    # addition as a launch of its own: only the down projection carries its residual there)
    assert calls["residual"] >= 2 * (steps - 1) * layers * (2 if batch == 2 else 1), calls
    assert batch == 2 or calls["gated"] >= 2 * (steps - 1) * layers, calls
    prompt = ref.sequences.shape[1] - steps
    agree = 0
    for t, (a, b) in enumerate(zip(out.scores, ref.scores)):
        if not torch.equal(out.sequences[:, : prompt + t], ref.sequences[:, : prompt + t]):
            break
        finite = torch.isfinite(b)
        assert torch.equal(torch.isfinite(a), finite)
        scale = b[finite].abs().max().item()
        diff = (a.float() - b.float())[finite].abs().max().item()
        assert diff <= 1e-2 * max(scale, 1.0), f"step {t}: scores differ by {diff} (scale {scale})"
        agree += 1
    print(f"llama: greedy paths agree for {agree} of {steps} steps; decode kernel calls {calls}", flush=True)
    assert agree >= 3


def test_models_built_one_after_the_other_do_not_share_fused_weights():
    """Two models of the same shapes, different weights, built and optimized one after the other with the first one
    freed in between: the allocator may give the second model the first one's parameter addresses, and the
    concatenated query/key/value weight kept for the first must not be served to the second."""
    import gc

    from kernl_amd.model_optimization import optimize_model

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q, self.k, self.v = (torch.nn.Linear(256, 256) for _ in range(3))

        def forward(self, x):
            return self.q(x) + 2.0 * self.k(x) - self.v(x)

    x = torch.randn((4, 128, 256), generator=torch.Generator().manual_seed(0)).half().cuda()
    for seed in (1, 2, 3):
        torch._dynamo.reset()
        torch.manual_seed(seed)
        model = Block().eval().half().cuda()
        with torch.inference_mode():
            expected = model(x).float().cpu()
        optimize_model(model)
        with torch.inference_mode():
            model(x)
            out = model(x).float().cpu()
        assert (out - expected).abs().max().item() < 2e-2, f"model {seed}: fused projection used stale weights"
        del model
        gc.collect()
        torch.cuda.empty_cache()


def test_weight_updates_after_capture_reach_the_fused_weights():
    """Weights written AFTER the model has been optimized and its hipGraph captured: the fused query/key/value weight
    aliases its parameters (any write, `param.data.copy_()` included, is seen by the next replay), the interleaved
    gate/value weight of a gated unit is rewritten in place before a replay when a version-counted write happened,
    and by `refresh_fused_parameters()` after a write the version counter does not see."""
    from kernl_amd.model_optimization import optimize_model
    from kernl_amd.optimizer.linear import refresh_fused_parameters

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q, self.k, self.v = (torch.nn.Linear(256, 256) for _ in range(3))
            self.gate, self.up = (torch.nn.Linear(256, 512, bias=False) for _ in range(2))
            self.down = torch.nn.Linear(512, 256, bias=False)

        def forward(self, x):
            h = self.q(x) + 2.0 * self.k(x) - self.v(x)
            return self.down(torch.nn.functional.silu(self.gate(h)) * self.up(h))

    torch._dynamo.reset()
    torch.manual_seed(0)
    model = Block().eval().half().cuda()
    twin = Block().eval().half().cuda()          # never optimized: says what the updated weights should give
    twin.load_state_dict(model.state_dict())
    x = torch.randn((4, 128, 256), generator=torch.Generator().manual_seed(0)).half().cuda()
    optimize_model(model)

    def check(what):
        with torch.inference_mode():
            out = model(x).float().cpu()
            expected = twin(x).float().cpu()
        err = (out - expected).abs().max().item()
        assert err < 2e-2 * max(1.0, expected.abs().max().item()), f"{what}: replay used stale weights (max abs err {err})"

    with torch.inference_mode():
        model(x)
    check("as captured")
    gen = torch.Generator().manual_seed(1)
    new_k = (torch.randn((256, 256), generator=gen) * 0.05).half().cuda()
    for m in (model, twin):
        m.k.weight.data.copy_(new_k)             # aliased: no version bump needed
    check("k.weight.data.copy_")
    new_gate = (torch.randn((512, 256), generator=gen) * 0.05).half().cuda()
    with torch.no_grad():
        for m in (model, twin):
            m.gate.weight.copy_(new_gate)        # version-counted write
    check("gate.weight.copy_")
    state = {k: (torch.randn(v.shape, generator=gen) * 0.05).half() for k, v in twin.state_dict().items()}
    twin.load_state_dict(state)
    model.load_state_dict(state)
    check("load_state_dict")
    for m in (model, twin):
        m.up.weight.data.mul_(0.5)               # invisible to the version counter
    assert refresh_fused_parameters() >= 1
    check("up.weight.data.mul_ + refresh_fused_parameters")
