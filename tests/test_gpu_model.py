"""The caller side: a Llama-shaped decoder (random weights) around the wave-index attention
(reference: model_hub/LLM.py:32-208).  With every cluster in the retrieval zone the wave-index
attention is exact, so the model must decode like the same model over a dense K/V cache."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _models(dev, device_positions=False, dt=torch.bfloat16):
    from retrievalattention_amd.model_hub import LlamaModel, LlamaShape
    shape = LlamaShape(hidden_size=256, intermediate_size=512, num_layers=2, num_heads=8, num_key_value_heads=2,
                       head_dim=128, vocab_size=1000)
    B, ctx, new = 2, 1024 + 68, 8
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, shape.vocab_size, (B, ctx), generator=g).to(dev)
    wave = LlamaModel(shape, ctx + new, dtype=dt, device=dev, seed=1)
    dense = LlamaModel(shape, ctx + new, dtype=dt, device=dev, seed=1)
    wave.init_kv_cache("RetroInfer", B, ctx, new, dict(n_centroids=64, n_segment=1, nprobe=64, max_compute_cluster_num=64),
                       device_positions=device_positions)
    dense.init_kv_cache("Full_Flash_Attn", B, ctx, new)
    return wave, dense, ids, new


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_full_probe_decodes_like_dense_attention(dev, dt):
    wave, dense, ids, new = _models(dev, dt=dt)
    lw, ld = wave.prefill_forward(ids), dense.prefill_forward(ids)
    assert torch.equal(lw, ld)               # prefill attention is the same dense kernel
    tok = ld.argmax(-1)
    for step in range(new - 1):
        lw, ld = wave.decode_forward(tok), dense.decode_forward(tok)
        torch.cuda.synchronize()
        d = (lw - ld).abs()
        assert float(d.max()) <= 5e-2 * max(1.0, float(ld.abs().max())), (step, float(d.max()))
        # (two bf16 models whose attention outputs differ in the last bits: logits agree to bf16 noise)
        assert float(d.mean()) <= 1.5e-2 * float(ld.abs().mean())
        tok = ld.argmax(-1)                  # both follow the dense model's tokens
    assert wave.kv_cache.context == dense.kv_cache.context == ids.shape[1] + new - 1


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_whole_token_replays_as_one_graph(dev, dt):
    """Every layer of a decoded token captured once, replayed for the following tokens."""
    wave, dense, ids, new = _models(dev, device_positions=True, dt=dt)
    lw, ld = wave.prefill_forward(ids), dense.prefill_forward(ids)
    tok_in = ld.argmax(-1).clone()
    # first decoded token eagerly on a side stream (warm-up for the capture), then capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        lw = wave.decode_forward(tok_in)
    torch.cuda.current_stream().wait_stream(side)
    ld = dense.decode_forward(tok_in)
    torch.cuda.synchronize()
    assert float((lw - ld).abs().max()) <= 5e-2 * max(1.0, float(ld.abs().max()))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = wave.decode_forward(tok_in)
    for step in range(new - 2):
        tok_in.copy_(ld.argmax(-1))
        graph.replay()
        wave.kv_cache.token_replayed()
        ld = dense.decode_forward(tok_in)
        torch.cuda.synchronize()
        d = (out - ld).abs()
        assert float(d.max()) <= 5e-2 * max(1.0, float(ld.abs().max())), (step, float(d.max()))
    assert wave.kv_cache.context == dense.kv_cache.context
    assert int(wave.position) == dense.kv_cache.context
