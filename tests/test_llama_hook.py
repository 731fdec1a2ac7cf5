"""Llama prefill hook (evaluate/llama/modify_sparse_attn.py in the package): host plumbing on the CPU, the prefill
path itself on the GPU.  The model is a tiny random-init Llama (no checkpoint is read)."""
import pytest
import torch

transformers = pytest.importorskip("transformers")

from evaluate.llama.modify_sparse_attn import set_mxfp_attn_llama, set_spas_sage_attn_llama  # noqa: E402


def _tiny_llama(dtype=torch.float32, head_dim=64):
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(vocab_size=128, hidden_size=4 * head_dim, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=head_dim, max_position_embeddings=1024)
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg).eval().to(dtype)


def test_hook_installs_and_decode_stays_on_sdpa():
    model = _tiny_llama()
    ids = torch.randint(0, 128, (1, 1), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        want = model(ids).logits
    assert set_spas_sage_attn_llama is set_mxfp_attn_llama
    set_mxfp_attn_llama(model, block_scale_type="diag")
    assert model.config._attn_implementation == "mxfp_attn"
    with torch.no_grad():
        got = model(ids).logits                      # q_len == 1: the reference's SDPA branch
    assert torch.equal(got, want)
    opts = [l.self_attn.mxfp_attn_options for l in model.model.layers]
    assert [o.layer_idx for o in opts] == [0, 1]
    assert all(o.decode_calls == 1 and o.prefill_calls == 0 for o in opts)


def test_prefill_on_cpu_fails_loudly():
    """No CPU fallback: a prefill with host tensors must raise, not silently run something else."""
    model = set_mxfp_attn_llama(_tiny_llama())
    ids = torch.randint(0, 128, (1, 160), generator=torch.Generator().manual_seed(2))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        with torch.no_grad():
            model(ids)


@pytest.mark.gpu
@pytest.mark.parametrize("head_dim,mode", [(128, "diag"), (64, "mxfp8")])
def test_prefill_and_generate_on_gpu(head_dim, mode):
    dev = "cuda:0"
    model = _tiny_llama(torch.bfloat16, head_dim).to(dev)
    ids = torch.randint(0, 128, (2, 384), generator=torch.Generator().manual_seed(3)).to(dev)
    with torch.no_grad():
        want = model(ids).logits.float()
    set_mxfp_attn_llama(model, block_scale_type=mode, verbose=True)
    with torch.no_grad():
        got = model(ids).logits.float()
        out = model.generate(ids[:1], max_new_tokens=4, do_sample=False)
    opts = [l.self_attn.mxfp_attn_options for l in model.model.layers]
    # forward + generate's prefill ran on the MXFP kernel, generate's 3 further steps on SDPA
    assert all(o.prefill_calls == 2 and o.decode_calls == 3 for o in opts), [(o.prefill_calls, o.decode_calls) for o in opts]
    for o in opts:                                   # against exact attention: quantization error only
        assert o.last_metric["Cossim"] >= 0.99, o.last_metric
    cos = torch.nn.functional.cosine_similarity(got.flatten(), want.flatten(), dim=0).item()
    assert cos >= 0.99, cos
    assert out.shape == (1, 388)
