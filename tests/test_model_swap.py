"""W2A8Linear as a swap-in for the linears of a Llama block.

Upstream's model-level caller loads a Hugging Face Llama in fp16 and calls ``generate``
(slimkernels/torch/llama.py:15-19, 34-43); its checkpoints are a download and unavailable here, so the
model below has that architecture at a small size with seeded random weights.  What is checked: the model
with its projections replaced by W2A8 layers against the same model holding the *dequantised* 2-bit weights
in fp16 -- the two differ only by the int8 activation quantisation and fp16 rounding, so their logits agree
closely; prefill (several token rows), batched rows, a single decode row (the fused one-launch path) and
greedy generation with a KV cache all run through the HIP kernels."""
import copy

import numpy as np
import pytest
import torch


def _tiny_llama():
    transformers = pytest.importorskip("transformers")
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=320, max_position_embeddings=128)
    torch.manual_seed(0)
    return transformers.LlamaForCausalLM(cfg).eval()


def _dequantised_copy(model, names, group_size, bits=2):
    """The model with each listed linear's weight replaced by what its 2- or 4-bit codes and fp16 scales stand for."""
    from slimkernels_amd.quantization import quantize_w2
    from slimkernels_amd.w4 import quantize_w4
    ref = copy.deepcopy(model)
    mods = dict(ref.named_modules())
    for name in names:
        lin = mods[name]
        w = lin.weight.detach().float().cpu().numpy()                 # [N, K]
        quantise, zero = (quantize_w2, 2.0) if bits == 2 else (quantize_w4, 8.0)
        codes, scales, _ = quantise(np.ascontiguousarray(w.T), group_size, "sym")   # [K, N], [G, N]
        s16 = scales.astype(np.float16).astype(np.float32)
        deq = (codes.astype(np.float32) - zero).reshape(-1, group_size, w.shape[0]) * s16[:, None, :]
        lin.weight.data = torch.from_numpy(np.ascontiguousarray(deq.reshape(w.shape[1], w.shape[0]).T)).to(lin.weight)
    return ref


def test_replace_linears_needs_the_model_on_the_gpu():
    from slimkernels_amd.torch import replace_linears
    model = torch.nn.Sequential(torch.nn.Linear(128, 64))
    with pytest.raises(ValueError, match="move the model to the GPU"):
        replace_linears(model)


def test_replace_linears_skips_what_it_cannot_take():
    from slimkernels_amd.torch import replace_linears

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.odd = torch.nn.Linear(100, 64)       # in_features not a multiple of the group size
            self.lm_head = torch.nn.Linear(128, 64)   # named in skip

    net = Net()
    assert replace_linears(net) == []
    assert isinstance(net.odd, torch.nn.Linear) and isinstance(net.lm_head, torch.nn.Linear)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,weight_only", [(2, False), (4, False), (2, True)])
def test_llama_block_with_w2a8_linears(gpu_ops, bits, weight_only):
    model = _tiny_llama().half().cuda()
    quant = copy.deepcopy(model)
    names = gpu_ops.replace_linears(quant, group_size=128, bits=bits, weight_only=weight_only)
    assert len(names) == 14 and "lm_head" not in names            # 7 projections x 2 layers
    layer_type = gpu_ops.W2A16Linear if weight_only else gpu_ops.W2A8Linear if bits == 2 else gpu_ops.W4A8Linear
    assert all(isinstance(dict(quant.named_modules())[n], layer_type) for n in names)
    ref = _dequantised_copy(model, names, 128, bits)

    g = torch.Generator().manual_seed(1)
    for shape in ((1, 12), (3, 5), (1, 1)):
        ids = torch.randint(0, 320, shape, generator=g).cuda()
        with torch.no_grad():
            want = ref(ids).logits.float()
            got = quant(ids).logits.float()
        err = (got - want).norm() / want.norm()
        print(f"tokens {shape}: relative L2 error of the logits {err:.4f}", flush=True)
        assert torch.isfinite(got).all()
        assert err < 0.03, f"tokens {shape}: logits off by {err:.4f}"

    ids = torch.randint(0, 320, (1, 6), generator=g).cuda()
    with torch.no_grad():
        out = quant.generate(ids, max_new_tokens=4, do_sample=False, pad_token_id=0)
    assert out.shape == (1, 10) and (out[:, :6] == ids).all()
