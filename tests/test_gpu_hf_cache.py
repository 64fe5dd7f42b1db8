"""The HF cache hook on a small random Llama: the packed cache + fused attention against the reference-style
fake-quantizing cache + dense attention, prefill and decode steps, with and without Med3x."""
import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not torch.cuda.is_available(), reason="needs a GPU")]
DEV = "cuda"


def tiny_llama(dtype):
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(vocab_size=256, hidden_size=512, intermediate_size=1024, num_hidden_layers=3, num_attention_heads=8,
                      num_key_value_heads=2, head_dim=64, max_position_embeddings=1024)
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg).to(dtype).to(DEV).eval()


@pytest.mark.parametrize("med3x", [False, True])
@pytest.mark.parametrize("dn", ["fp16", "bf16"])
def test_packed_cache_matches_fake_quant_cache(dn, med3x):
    import hqmq
    from transformers import DynamicCache
    from src.model_utils import ATTN_NAME, PackedQuantizedCache, QuantizedCache
    dt = {"fp16": torch.float16, "bf16": torch.bfloat16}[dn]
    model = tiny_llama(dt)
    q = hqmq.HQMQ(n_layers=3, n_heads=2, secondary_size=96, radius_bits=4, device=DEV)
    if med3x:
        q = hqmq.with_outlier_extraction(q, C=3.0)
        with torch.no_grad():                      # outlier channels: two chunks of K and one of V per KV head
            for layer in model.model.layers:
                layer.self_attn.k_proj.weight[8:16] *= 12.0
                layer.self_attn.k_proj.weight[64 + 20:64 + 24] *= 12.0
                layer.self_attn.v_proj.weight[40:44] *= 12.0
    ids = torch.randint(0, 256, (2, 150), generator=torch.Generator().manual_seed(1)).to(DEV)
    steps = 6

    def run(cache):
        logits = []
        with torch.no_grad():
            out = model(ids[:, :-steps], past_key_values=cache, use_cache=True)
            logits.append(out.logits[:, -1].float())
            for s in range(steps):
                out = model(ids[:, -steps + s:ids.shape[1] - steps + s + 1], past_key_values=cache, use_cache=True)
                logits.append(out.logits[:, -1].float())
        return torch.stack(logits)

    model.set_attn_implementation("sdpa")
    want = run(QuantizedCache(q))                      # reference behaviour: fake-quantized dense cache
    plain = run(DynamicCache())                        # unquantized, to size the effect of quantization
    model.set_attn_implementation(ATTN_NAME)
    packed = PackedQuantizedCache(q, max_tokens=256, sideband_frac=0.5)    # the planted channels flag ~20 % of K chunks
    got = run(packed)
    packed.check_overflow()
    assert packed.get_seq_length() == ids.shape[1]
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    quant_effect = (want - plain).abs().max().item()
    # the two paths hold the same codes; they differ by the decode rounding convention (<= 1 ulp of the cache
    # dtype) and by fp16-vs-cache-dtype products inside attention, far less than quantization itself moves the logits
    print(f"{dn} med3x={med3x}: max|logit| {scale:.3f}, packed vs fake-quant {err:.2e}, quantized vs unquantized {quant_effect:.2e}")
    assert err < (0.02 if dn == "fp16" else 0.06) * scale and err < 0.5 * quant_effect, (err, scale, quant_effect)
    if med3x:
        assert all(int(layer.packed.K.sb_count.sum()) > 0 and int(layer.packed.V.sb_count.sum()) > 0 for layer in packed.layers)
    # compressed size: 4 bits/value of codes + the per-token scale (+ flags and sideband with Med3x)
    dense_bytes = 3 * 2 * 2 * 2 * ids.shape[1] * 64 * 2
    assert packed.nbytes() < (0.6 if med3x else 0.36) * dense_bytes


@pytest.mark.parametrize("med3x", [False, True])
@pytest.mark.parametrize("dn", ["fp16", "bf16"])
def test_attention_inside_the_model_meets_the_kernel_bound(dn, med3x, monkeypatch):
    """Parity of the attention calls the model itself makes: every decode-step call of the fused kernel inside the HF
    forward pass (real activations: RoPE'd queries, the layers' own K / V with planted outlier channels) is checked
    against two fp32 references computed from the codes in that layer's packed cache, with the bound the kernel is
    held to everywhere else (tests/helpers.py:assert_attention_close)."""
    import hqmq
    import hqmq_amd.hf_cache as hf
    from hqmq_amd import ops
    from src.model_utils import ATTN_NAME, PackedQuantizedCache
    from tests.helpers import assert_attention_close, exact_dense, gpu_attention_refs
    dt = {"fp16": torch.float16, "bf16": torch.bfloat16}[dn]
    model = tiny_llama(dt)
    q = hqmq.HQMQ(n_layers=3, n_heads=2, secondary_size=96, radius_bits=4, device=DEV)
    if med3x:
        q = hqmq.with_outlier_extraction(q, C=3.0)
        with torch.no_grad():
            for layer in model.model.layers:
                layer.self_attn.k_proj.weight[8:16] *= 12.0
                layer.self_attn.v_proj.weight[40:44] *= 12.0
    calls = []
    inner = hf.fused_attention_packed

    def recording(query, cache, **kw):
        out = inner(query, cache, **kw)
        if query.shape[2] == 1:
            calls.append((query.clone(), cache, kw["T_kv"], out.clone()))
        return out
    monkeypatch.setattr(hf, "fused_attention_packed", recording)
    ids = torch.randint(0, 256, (2, 150), generator=torch.Generator().manual_seed(5)).to(DEV)
    model.set_attn_implementation(ATTN_NAME)
    cache = PackedQuantizedCache(q, max_tokens=256, sideband_frac=0.5)
    with torch.no_grad():
        model(ids[:, :147], past_key_values=cache, use_cache=True)
        for t in range(147, 150):
            model(ids[:, t:t + 1], past_key_values=cache, use_cache=True)
    cache.check_overflow()
    assert len(calls) == 9                                      # three layers, three decode steps
    worst = 0.0
    for query, packed, L, out in calls:
        K_D, V_D = ops.dequant_packed(packed.K, L, 0), ops.dequant_packed(packed.V, L, 0)
        for b in range(query.shape[0]):
            # flagged chunks are verbatim in the dense decode: it serves as the source of their exact values
            K_x, V_x = exact_dense(packed.K, b, L, K_D[b]), exact_dense(packed.V, b, L, V_D[b])
            ref_d, ref_x, a_abs = gpu_attention_refs(query[b, :, 0], K_D[b].float(), V_D[b].float(), K_x, V_x)
            worst = max(worst, assert_attention_close(out[b, :, 0], ref_d.cpu(), ref_x.cpu(), a_abs.cpu(), base=2e-3,
                                                      what=f"{dn} med3x={med3x} L={L} sequence {b}"))
    print(f"\n{dn} med3x={med3x}: attention calls inside the model, max |O - ref_D| {worst:.3e}")


def test_packed_cache_crop_replays_identically():
    """Rolling the packed cache back (speculative decoding) and decoding the same tokens again gives the same logits
    bit for bit, with outliers on both sides of the cut."""
    import hqmq
    from src.model_utils import ATTN_NAME, PackedQuantizedCache
    model = tiny_llama(torch.float16)
    q = hqmq.with_outlier_extraction(hqmq.HQMQ(n_layers=3, n_heads=2, secondary_size=96, radius_bits=4, device=DEV), C=3.0)
    with torch.no_grad():
        for layer in model.model.layers:
            layer.self_attn.k_proj.weight[8:16] *= 12.0
            layer.self_attn.v_proj.weight[40:44] *= 12.0
    ids = torch.randint(0, 256, (2, 150), generator=torch.Generator().manual_seed(2)).to(DEV)
    model.set_attn_implementation(ATTN_NAME)
    cache = PackedQuantizedCache(q, max_tokens=256, sideband_frac=0.5)

    def decode(first, last):
        with torch.no_grad():
            return torch.stack([model(ids[:, t:t + 1], past_key_values=cache, use_cache=True).logits[:, -1].float()
                                for t in range(first, last)])
    with torch.no_grad():
        model(ids[:, :139], past_key_values=cache, use_cache=True)
    once = decode(139, 146)
    counts = [int(layer.packed.K.sb_count.sum()) for layer in cache.layers]
    cache.crop(-5)
    assert cache.get_seq_length() == 141
    assert all(int(layer.packed.K.sb_count.sum()) < c for layer, c in zip(cache.layers, counts))
    again = decode(141, 146)
    cache.check_overflow()
    assert cache.get_seq_length() == 146 and torch.equal(once[2:], again)
    assert [int(layer.packed.K.sb_count.sum()) for layer in cache.layers] == counts


def test_left_padded_generation_batch():
    """Sequences of different lengths, left-padded as generate() lays them out: the packed cache + fused attention
    follow the fake-quantizing cache + sdpa on the real positions, prefill and decode steps."""
    import hqmq
    from src.model_utils import ATTN_NAME, PackedQuantizedCache, QuantizedCache
    dt = torch.float16
    model = tiny_llama(dt)
    q = hqmq.HQMQ(n_layers=3, n_heads=2, secondary_size=96, radius_bits=4, device=DEV)
    B, T, steps = 3, 90, 4
    pads = [0, 13, 40]
    ids = torch.randint(1, 256, (B, T + steps), generator=torch.Generator().manual_seed(3)).to(DEV)
    mask = torch.ones(B, T + steps, dtype=torch.long, device=DEV)
    for b, p in enumerate(pads):
        mask[b, :p] = 0
        ids[b, :p] = 0
    pos = (mask.cumsum(-1) - 1).clamp(min=0)

    def run(cache):
        logits = []
        with torch.no_grad():
            out = model(ids[:, :T], attention_mask=mask[:, :T], position_ids=pos[:, :T], past_key_values=cache, use_cache=True)
            logits.append(out.logits[:, -1].float())
            for s in range(steps):
                out = model(ids[:, T + s:T + s + 1], attention_mask=mask[:, :T + s + 1], position_ids=pos[:, T + s:T + s + 1],
                            past_key_values=cache, use_cache=True)
                logits.append(out.logits[:, -1].float())
        return torch.stack(logits)

    model.set_attn_implementation("sdpa")
    want = run(QuantizedCache(q))
    model.set_attn_implementation(ATTN_NAME)
    packed = PackedQuantizedCache(q, max_tokens=128)
    got = run(packed)
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    print(f"left-padded batch: max|logit| {scale:.3f}, packed vs fake-quant {err:.2e}")
    assert err < 0.02 * scale, (err, scale)
