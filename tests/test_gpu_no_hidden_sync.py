"""Steady-state steps of every layer type under torch's synchronisation debug mode: once the statistics are
frozen no call of a step may synchronise the host with the device (a pageable host-to-device copy, an
`.item()`, a `nonzero`).  The only wait of a step is the one on the event behind the attention map's
kept-entry count, which torch does not count as a synchronising call and which waits for work enqueued long
before."""
import warnings

import pytest
import torch

import test_gpu_layers as TL
import test_gpu_roberta as TR

pytestmark = pytest.mark.gpu


def synchronising_calls(make, run, t):
    layer = make()
    for _ in range(4):                               # past calibration (threshold 2) and past the first frozen step
        run(layer, t).backward(t.grad)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("warn")
    try:
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            for _ in range(2):
                run(layer, t).backward(t.grad)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    torch.cuda.synchronize()
    return [f"{w.filename.rsplit('/', 1)[-1]}:{w.lineno}: {w.message}" for w in caught if "synchroniz" in str(w.message).lower()]


@pytest.mark.parametrize("layer_type", ["baseline", "intra", "intra_inter", "intra_inter_full_fuse"])
@pytest.mark.parametrize("family", ["llama", "mistral", "llama_flash_attn"])
def test_decoder_layer_steps_do_not_synchronise(dev, family, layer_type):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import llama, llama_flash_attn, mistral
    pkg = {"llama": llama, "mistral": mistral, "llama_flash_attn": llama_flash_attn}[family]
    t = TL.make_layer_inputs(dev, 1, B=2, S=128, hidden=1024, heads=8, kv_heads=2 if family == "mistral" else 8, inter=2816)
    cfg = TL.config(layer_type, 4, sm_ratio=0.05, thr=2)
    make = {"llama": llama.make_fused_llama_layer, "mistral": mistral.make_fused_mistral_layer,
            "llama_flash_attn": llama_flash_attn.make_fused_llama_layer}[family]
    run = (lambda l, tt: TL.run_fused(l, tt, use_mask=False)) if family == "llama_flash_attn" else TL.run_fused
    found = synchronising_calls(lambda: make(cfg), run, t)
    assert not found, f"{pkg.__name__} {layer_type}: {found}"


@pytest.mark.parametrize("layer_type", ["baseline", "intra", "intra_inter"])
def test_encoder_layer_steps_do_not_synchronise(dev, layer_type):
    import hyclora_amd  # noqa: F401
    from hyclora_amd.models import roberta
    t = TR.make_inputs(dev, 3, B=2, S=128, hidden=768, heads=12, inter=3072)
    found = synchronising_calls(lambda: roberta.make_fused_roberta_layer(TL.config(layer_type, 4, sm_ratio=0.05, thr=2)),
                                TR.run_fused, t)
    assert not found, f"roberta {layer_type}: {found}"


def test_nf4_weights_do_not_synchronise(dev):
    """A layer on NF4 frozen weights whose quant state carries no code book: the default table must already be
    on the device (it used to be copied from the host at every dequantisation)."""
    import hyclora_amd  # noqa: F401
    from hyclora_amd.operators import nf4
    packed = torch.randint(0, 256, (64 * 128 // 2, 1), device=dev, dtype=torch.uint8)
    qs = nf4.make_quant_state(torch.rand(64 * 128 // 64, device=dev), (64, 128), blocksize=64)
    nf4.dequantize_nf4(packed, qs)                   # first call may upload the table
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("warn")
    try:
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            for _ in range(3):
                nf4.dequantize_nf4(packed, qs)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert not [w for w in caught if "synchroniz" in str(w.message).lower()]


def test_the_debug_mode_sees_a_synchronising_call(dev):
    """Positive control: a read-back under the same mode is reported, so the tests above can fail."""
    x = torch.ones(4, device=dev)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("warn")
    try:
        with warnings.catch_warnings(record=True) as caught:
            warnings.simplefilter("always")
            x.sum().item()
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert [w for w in caught if "synchroniz" in str(w.message).lower()]
