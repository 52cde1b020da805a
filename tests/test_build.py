"""The in-tree native libraries build for gfx950 and load on a CPU-only host
(catches undefined symbols, e.g. a template kernel whose host stub was never
instantiated, before anything reaches a GPU box)."""
import torch

from replisense_rfq_amd import _build, runtime


def test_native_libraries_build_and_load():
    so = _build.build_kernels()
    torch.ops.load_library(str(so))
    for op in ("rms_norm", "attn_decode", "attn_prefill", "skinny_gemm", "moe_skinny",
               "moe_grouped_gemm", "car_allreduce", "sample_partial"):
        assert hasattr(torch.ops.rfq_amd, op), op
    rt = runtime.load()
    assert hasattr(rt, "EngineCore") and hasattr(rt, "Grammar")


def test_layer_list_kernel_library_builds_and_loads():
    so = _build.build_mix_kernels()
    torch.ops.load_library(str(so))
    for op in ("embed_sinusoid", "sandwich_norm", "canon_conv", "head_norm_append",
               "attn_talk_decode", "attn_mixq_prefill", "attn_mix_mfma", "glu_clamped",
               "mixq_mfma_ok", "qk_norm_rotary_append", "attn_keep_window", "xielu_rows",
               "keep_mfma_ok"):
        assert hasattr(torch.ops.rfq_mix, op), op
    assert torch.ops.rfq_mix.keep_mfma_ok(128, 128, 32, False)
    assert torch.ops.rfq_mix.keep_mfma_ok(576, 512, 32, True)
    assert not torch.ops.rfq_mix.keep_mfma_ok(48, 48, 32, False)
    assert torch.ops.rfq_mix.mixq_mfma_ok(32, 8, 128, 128, 32)
    assert not torch.ops.rfq_mix.mixq_mfma_ok(6, 3, 24, 40, 32)
