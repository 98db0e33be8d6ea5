"""CPU-side checks of the boundary: the C-ABI library loads and exports every symbol
include/samfast.h declares (no compute calls without a GPU); the Python mirror keeps the
reference's names and signatures; the product refuses to run without its kernels."""

import ctypes
import inspect
import re
from pathlib import Path

import pytest
import torch
import torch.nn as nn

ROOT = Path(__file__).resolve().parents[1]


def _header_functions(header="samfast.h"):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(samfast_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    """include/samfast.h is the path's boundary; include/samfast_bench.h holds the measurement
    aids.  The library exports exactly what the two declare and the Python binding mirrors both."""
    from samfast_amd import _lib
    names = _header_functions()
    assert len(names) >= 8
    assert not [n for n in names if n.startswith("samfast_bench_")]
    bench = _header_functions("samfast_bench.h")
    assert bench and all(n.startswith("samfast_bench_") for n in bench)
    lib = ctypes.CDLL(str(_lib.lib_path()))
    for n in names + bench:
        assert hasattr(lib, n), n
    assert sorted(_lib.EXPORTED_SYMBOLS) == names
    assert sorted(_lib.BENCH_SYMBOLS) == bench
    loaded = _lib.load()
    assert loaded.samfast_version() == 1
    assert loaded.samfast_arch() == b"gfx950"


def test_knobs_are_named_and_bounded_without_gpu():
    """The variant knobs take the documented names only; the bare matrix-instruction loops refuse
    launches that would hold the GPU for more than about a second (checked before any launch)."""
    from samfast_amd import _lib
    lib = _lib.load()
    assert lib.samfast_bench_set_knob(b"SAMFAST_GEMM_PERSIST", 1, 0) == 0
    assert lib.samfast_bench_set_knob(b"SAMFAST_GEMM_PERSIST", 0, 1) == 0
    assert lib.samfast_bench_set_knob(b"SAMFAST_NO_SUCH_KNOB", 1, 0) == -1
    assert b"unknown knob" in lib.samfast_last_error()
    # every knob the bench header and the internal enumeration name is known to the library, and they
    # name the same set
    import re
    root = Path(__file__).resolve().parents[1]
    documented = set(re.findall(r"SAMFAST_(?:GEMM|ATTN|SPARSE)_[A-Z0-9_]+", (root / "include" / "samfast_bench.h").read_text()))
    internal = set(re.findall(r"// (SAMFAST_[A-Z0-9_]+):", (root / "segment-anything-fast_amd" / "csrc" / "samfast_internal.hpp").read_text()))
    assert documented == internal and len(documented) >= 11, documented ^ internal
    for name in sorted(documented):
        assert lib.samfast_bench_set_knob(name.encode(), 0, 1) == 0, name
    buf = ctypes.create_string_buffer(65536)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    assert lib.samfast_bench_mfma_ceiling(0, p, 1 << 20, 1 << 24, None, p, None) == -1
    assert b"2^27" in lib.samfast_last_error()
    assert lib.samfast_bench_mfma_valu_overlap(0, p, 1 << 12, 1 << 20, 0, p, None) == -1
    assert b"2^27" in lib.samfast_last_error()


def test_fused_quant_gemm_refuses_outputs_its_quantiser_cannot_address():
    """lin1-shaped call with M * N >= 2^31: the in-kernel quantiser's 32-bit offsets would wrap, so
    the entry point (and its allocation-free form) refuses before anything is launched."""
    from samfast_amd import _lib
    lib = _lib.load()
    M, N, K = 900000, 5120, 1280  # M * K < 2^31 <= M * N
    args = [None, None, None, None, None, None, N, M, N, K, 0, 1, None, 0, 1, None, None, 0.0, None, None, 1]
    assert lib.samfast_gemm_i8_fused_quant(*args, None, None) == -1
    assert b"2^31" in lib.samfast_last_error()
    assert lib.samfast_gemm_i8_fused_quant_noalloc(*args, None) == -1
    assert b"2^31" in lib.samfast_last_error()


def test_empty_calls_are_no_ops_without_gpu():
    """No rows / no images: every entry point validates the shape, launches nothing and returns 0,
    also with null row buffers (what an empty tensor hands over); a negative count is an error."""
    from samfast_amd import _lib
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    assert lib.samfast_quant_rowwise_i8(None, 256, None, None, 0, 256, 0, 0, None) == 0
    assert lib.samfast_quant_rowwise_i8(None, 256, None, None, 0, 256, 0, 1, None) == 0
    assert lib.samfast_layernorm_quant_i8(None, 256, p, p, 1e-6, None, None, None, 0, 256, 0, 0, None) == 0
    assert lib.samfast_gemm_i8_i32(None, p, None, 0, 64, 256, None) == 0
    assert lib.samfast_gemm_i8_scale_bias(None, None, p, p, None, None, 64, 0, 64, 256, 0, None) == 0
    assert lib.samfast_gemm_i8_fused(None, None, p, p, p, None, 64, 0, 64, 256, 0, 2, None, 64, None, 1, None) == 0
    assert lib.samfast_gemm_i8_sparse24_i32(None, p, p, None, 0, 64, 256, None) == 0
    assert lib.samfast_gemm_i8_sparse24_fused(None, None, p, p, p, None, None, 64, 0, 64, 256, 0, 1, None, 0, 0, None) == 0
    strides = [64] * 12
    assert lib.samfast_attn_relpos_fwd(None, None, None, None, None, None, 0, 12, 64, 64, 64,
                                       *strides, 0, 0.125, None) == 0
    assert lib.samfast_attn_relpos_bias_fwd(None, None, None, None, None, None, 0, 12, 14, 14, 80,
                                            *([80] * 12), *([16] * 6), 0, 0.1, None) == 0
    # the shape is still checked
    assert lib.samfast_quant_rowwise_i8(None, 256, None, None, -1, 256, 0, 0, None) == -1
    assert lib.samfast_gemm_i8_i32(None, p, None, 0, 64, 100, None) == -1
    assert lib.samfast_attn_relpos_fwd(None, None, None, None, None, None, 0, 12, 64, 64, 48,
                                       *strides, 0, 0.125, None) == -2
    assert lib.samfast_attn_relpos_fwd(None, None, None, None, None, None, -1, 12, 64, 64, 64,
                                       *strides, 0, 0.125, None) == -1


def test_argument_validation_without_gpu():
    """Validation runs on the host before any launch, so error codes are testable here."""
    from samfast_amd import _lib
    lib = _lib.load()
    rc = lib.samfast_gemm_i8_i32(None, None, None, 16, 16, 64, None)
    assert rc == -1 and b"null pointer" in lib.samfast_last_error()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    rc = lib.samfast_gemm_i8_i32(p, p, p, 16, 16, 100, None)
    assert rc == -1 and b"multiple of 64" in lib.samfast_last_error()
    rc = lib.samfast_quant_rowwise_i8(p, 12, p, p, 4, 12, 0, 0, None)
    assert rc == -1 and b"multiple of 8" in lib.samfast_last_error()
    rc = lib.samfast_quant_rowwise_i8(p, 96, p, p, 4, 96, 0, 1, None)  # K-block major needs K % 64 == 0
    assert rc == -1 and b"K-block major" in lib.samfast_last_error()
    rc = lib.samfast_gemm_i8_fused(p, p, p, p, None, p, 64, 4, 64, 256, 0, 0, None, 0, None, 7, None)
    assert rc == -1 and b"layout" in lib.samfast_last_error()
    strides = [0] * 12
    rc = lib.samfast_attn_relpos_fwd(p, p, p, p, p, p, 1, 1, 10, 10, 48, *strides, 0, 0.125, None)
    assert rc == -2 and b"head_dim" in lib.samfast_last_error()
    rc = lib.samfast_attn_relpos_fwd(p, p, p, p, p, p, 1, 1, 20, 20, 64, *([64] * 12), 0, 0.125, None)
    assert rc == -2 and b"neither" in lib.samfast_last_error()
    rc = lib.samfast_attn_relpos_fwd(p, p, p, p, p, p, 1, 1, 14, 14, 64, *([64] * 12), 2, 0.125, None)
    assert rc == -2 and b"element type" in lib.samfast_last_error()  # neither SAMFAST_BF16 nor SAMFAST_F16
    rc = lib.samfast_quant_rowwise_i8(p, 64, p, p, 4, 64, 1, 0, None)
    assert rc == -2  # the linears are bf16 only


def test_ops_refuse_cpu_tensors():
    from samfast_amd import ops
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.quant_rowwise(x)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.gemm_i8_i32(torch.zeros(4, 64, dtype=torch.int8), torch.zeros(8, 64, dtype=torch.int8))


def test_registry_surface():
    import samfast_amd
    for reg in (samfast_amd.sam_model_registry, samfast_amd.sam_model_fast_registry):
        assert set(reg) == {"default", "vit_h", "vit_l", "vit_b"}
    sig = inspect.signature(samfast_amd.build_sam_fast_vit_h)
    assert list(sig.parameters) == ["checkpoint", "compile_mode", "dtype"]
    assert sig.parameters["compile_mode"].default == "max-autotune"
    assert sig.parameters["dtype"].default == torch.bfloat16
    sam = samfast_amd.sam_model_fast_registry["vit_b"]()
    assert next(sam.image_encoder.parameters()).dtype == torch.bfloat16 and not sam.image_encoder.training
    pred = samfast_amd.SamPredictor(sam)
    assert pred.is_image_set is False
    img = torch.zeros(1, 3, 512, 1024)
    assert sam.preprocess(img).shape == (1, 3, 1024, 1024)


def test_fast_registry_wraps_the_encoder_for_graph_replay():
    """compile_mode of the fast builders (build_sam.py:67-71 of the reference compiles the encoder
    with it): any mode wraps the encoder for HIP-graph replay, None leaves it bare.  The wrapper
    forwards attributes, keeps the reference's post-compile state-dict prefix and drops its
    recordings whenever weights or modules are replaced."""
    import samfast_amd
    from samfast_amd import tools
    from samfast_amd.graphs import ReplayedEncoder
    from samfast_amd.modeling import ImageEncoderViT
    sam = samfast_amd.sam_model_fast_registry["vit_b"]()
    enc = sam.image_encoder
    assert isinstance(enc, ReplayedEncoder) and enc.compile_mode == "max-autotune"
    assert enc.img_size == 1024 and len(enc.blocks) == 12 and isinstance(enc._orig_mod, ImageEncoderViT)
    assert all(k.startswith("_orig_mod.") for k in enc.state_dict())
    bare = samfast_amd.sam_model_fast_registry["vit_b"](compile_mode=None).image_encoder
    assert isinstance(bare, ImageEncoderViT)
    assert not enc.replays(torch.zeros(1, 3, 1024, 1024))  # CPU tensors run eagerly
    for mutate in (lambda: tools.replace_with_custom_fn_if_matches_filter(enc, lambda m: m, lambda m, f: False),
                   lambda: enc.load_state_dict(enc.state_dict()),
                   lambda: samfast_amd.apply_fake_sparsity(sam, lambda m, f: False),
                   lambda: enc.float()):
        enc._graphs["stale"] = object()
        mutate()
        assert not enc._graphs


def test_module_signatures_follow_reference():
    from samfast_amd.modeling import Attention, Block, ImageEncoderViT, MLPBlock
    assert list(inspect.signature(Attention.__init__).parameters)[1:] == [
        "dim", "num_heads", "qkv_bias", "use_rel_pos", "rel_pos_zero_init", "input_size"]
    assert list(inspect.signature(MLPBlock.__init__).parameters)[1:] == ["embedding_dim", "mlp_dim", "act"]
    assert list(inspect.signature(Block.__init__).parameters)[1:] == [
        "dim", "num_heads", "mlp_ratio", "qkv_bias", "norm_layer", "act_layer", "use_rel_pos",
        "rel_pos_zero_init", "window_size", "input_size"]
    att = Attention(64, 2, use_rel_pos=True, input_size=(14, 14))
    assert {n for n, _ in att.named_parameters()} == {
        "qkv.weight", "qkv.bias", "proj.weight", "proj.bias", "rel_pos_h", "rel_pos_w"}
    assert att.rel_pos_h.shape == (27, 32)
    enc_sig = inspect.signature(ImageEncoderViT.__init__)
    assert enc_sig.parameters["window_size"].default == 0 and enc_sig.parameters["embed_dim"].default == 768


def test_swap_helpers():
    from samfast_amd import Int8DynamicLinear, apply_dynamic_quant
    from samfast_amd.tools import replace_with_custom_fn_if_matches_filter
    from samfast_amd.modeling import Block
    blk = Block(64, 2, use_rel_pos=True, window_size=3, input_size=(8, 8))
    seen = []
    replace_with_custom_fn_if_matches_filter(
        blk, lambda m: m, lambda m, fqn: (seen.append(fqn) or False))
    assert {"norm1", "attn", "attn.qkv", "attn.proj", "norm2", "mlp", "mlp.lin1", "mlp.lin2", "mlp.act"} <= set(seen)
    w = blk.mlp.lin1.weight.detach().clone()
    apply_dynamic_quant(blk, lambda m, fqn: fqn.startswith("mlp."))
    assert isinstance(blk.mlp.lin1, Int8DynamicLinear) and isinstance(blk.mlp.lin2, Int8DynamicLinear)
    assert isinstance(blk.attn.qkv, nn.Linear)
    assert blk.mlp.lin1.wq.dtype == torch.int8 and blk.mlp.lin1.sw.dtype == torch.float32
    assert (blk.mlp.lin1.weight - w).abs().max() <= blk.mlp.lin1.sw.max() * 0.5001
    blk = blk.to(torch.bfloat16)  # scales and integer weights survive a dtype cast untouched
    assert blk.mlp.lin1.sw.dtype == torch.float32 and blk.mlp.lin1.wq.dtype == torch.int8
    with pytest.raises(RuntimeError, match="GPU"):
        blk.mlp(torch.zeros(1, 8, 8, 64, dtype=torch.bfloat16))  # no CPU route for the int8 path


def test_composite_cpu_route_is_the_reference_fallback():
    """fp32 / CPU inputs take the eager SDPA route exactly as flash_4.py:368-370."""
    from samfast_amd.flash_4 import _attention_rel_h_rel_w
    from oracle import relpos_attention as ora
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 2, 196, 64, generator=g) for _ in range(3))
    rel_h, rel_w = torch.randn(1, 2, 196, 14, 1, generator=g), torch.randn(1, 2, 196, 1, 14, generator=g)
    got = _attention_rel_h_rel_w(q, k, v, rel_h, rel_w)
    assert torch.allclose(got, ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w), atol=1e-5)
    assert hasattr(torch.ops.customflash, "custom_flash_aligned")


def test_checkpoint_with_reference_key_names_loads(tmp_path):
    """A checkpoint in the layout the released SAM files have (key names follow the module
    tree of the reference, modeling/image_encoder.py:15-120 and modeling/sam.py:18-58; prompt
    encoder and mask decoder entries present) loads through the registry, and the quantised
    modules are then built from the loaded weights."""
    import samfast_amd
    from samfast_amd import Int8DynamicLinear, apply_dynamic_quant
    donor = samfast_amd.sam_model_registry["vit_b"]()
    g = torch.Generator().manual_seed(11)
    sd = {}
    for k, v in donor.state_dict().items():
        sd[k] = (torch.randn(v.shape, generator=g) * 0.02).to(torch.float16) if v.is_floating_point() else v
    # what the module tree of the reference's encoder gives, written out by rule
    expect = {"image_encoder.pos_embed", "image_encoder.patch_embed.proj.weight", "image_encoder.patch_embed.proj.bias",
              "image_encoder.neck.0.weight", "image_encoder.neck.1.weight", "image_encoder.neck.1.bias",
              "image_encoder.neck.2.weight", "image_encoder.neck.3.weight", "image_encoder.neck.3.bias"}
    for i in range(12):
        for leaf in ("norm1.weight", "norm1.bias", "attn.rel_pos_h", "attn.rel_pos_w", "attn.qkv.weight",
                     "attn.qkv.bias", "attn.proj.weight", "attn.proj.bias", "norm2.weight", "norm2.bias",
                     "mlp.lin1.weight", "mlp.lin1.bias", "mlp.lin2.weight", "mlp.lin2.bias"):
            expect.add(f"image_encoder.blocks.{i}.{leaf}")
    assert {k for k in sd if k.startswith("image_encoder.")} == expect
    # entries of the parts that are not built here
    sd["prompt_encoder.pe_layer.positional_encoding_gaussian_matrix"] = torch.zeros(2, 128)
    sd["mask_decoder.iou_token.weight"] = torch.zeros(1, 256)
    path = tmp_path / "sam_vit_b.pth"
    torch.save(sd, path)
    sam = samfast_amd.sam_model_registry["vit_b"](checkpoint=str(path))
    w = sam.image_encoder.blocks[3].mlp.lin1.weight
    assert torch.equal(w, sd["image_encoder.blocks.3.mlp.lin1.weight"].float())
    assert sam.image_encoder.blocks[0].attn.rel_pos_h.shape == (27, 64)     # windowed block: 2*14-1
    assert sam.image_encoder.blocks[2].attn.rel_pos_h.shape == (127, 64)    # global block: 2*64-1
    apply_dynamic_quant(sam.image_encoder.blocks[3])
    q = sam.image_encoder.blocks[3].mlp.lin1
    assert isinstance(q, Int8DynamicLinear)
    assert (q.weight - w).abs().max() <= q.sw.max() * 0.5001


def test_attention_wrappers_reject_mismatched_shapes_before_any_launch():
    """The library is only told the grid; it would walk gh*gw tokens of every (batch, head) slice
    whatever the tensors hold.  The wrappers therefore pin every shape on the host - these raise
    on CPU tensors, i.e. before the device check and before anything could be launched."""
    from samfast_amd import flash_4, ops
    bf = torch.bfloat16
    q = torch.zeros(1, 2, 2048, 64, dtype=bf)
    tabs = torch.zeros(127, 64, dtype=bf)
    with pytest.raises(RuntimeError, match="must be"):            # 2048 tokens on a 64x64 grid
        ops.attn_relpos(q, q, q, tabs, tabs, (64, 64))
    q4 = torch.zeros(1, 2, 4096, 64, dtype=bf)
    with pytest.raises(RuntimeError, match="shape of q"):
        ops.attn_relpos(q4, q4[:, :, :2048], q4, tabs, tabs, (64, 64))
    with pytest.raises(RuntimeError, match="dtype of q"):
        ops.attn_relpos(q4, q4.float(), q4, tabs, tabs, (64, 64))
    with pytest.raises(RuntimeError, match="out must"):
        ops.attn_relpos(q4, q4, q4, tabs, tabs, (64, 64), out=torch.zeros(1, 2, 2048, 64, dtype=bf))
    rel_h = torch.zeros(1, 2, 2048, 64, dtype=bf)
    with pytest.raises(RuntimeError, match="must be"):            # bias says 64x64 keys, q has 2048 tokens
        ops.attn_relpos_bias(q, q, q, rel_h, rel_h)
    with pytest.raises(RuntimeError, match="bias factors"):       # bias rows do not match q's tokens
        ops.attn_relpos_bias(q4, q4, q4, rel_h, torch.zeros(1, 2, 4096, 64, dtype=bf))
    with pytest.raises(RuntimeError, match="must be"):
        ops.attn_relpos_windowed(q, q, q, torch.zeros(27, 64, dtype=bf), torch.zeros(27, 64, dtype=bf),
                                 torch.zeros(2, 64, dtype=bf), torch.zeros(2, 64, dtype=bf), (64, 64), 14, 0.125)
    # the registered operator derives the key grid from the token count: 64-wide rows only
    with pytest.raises(RuntimeError, match="64-wide key grid"):
        flash_4._custom_flash_aligned_gpu(q[:, :, :2000], q[:, :, :2000], q[:, :, :2000],
                                          torch.zeros(1, 2, 2000, 128, dtype=bf), 0.125)
    # a consistent call gets as far as the device check
    with pytest.raises(RuntimeError, match="GPU"):
        ops.attn_relpos(q4, q4, q4, tabs, tabs, (64, 64))


def test_weight_quantiser_conventions_closed_form():
    """The default per-channel convention (absmax / 127, clamp +-127) and torchao's
    (absmax / 127.5 clamped at float32 eps, clamp -128..127, arithmetic in the weight's dtype),
    on values whose quotients are exact."""
    from samfast_amd.quant import quantize_weight_per_channel
    w = torch.tensor([[127.0, -63.5, 1.0, 0.0], [-255.0, 255.0, 2.0, -1.0], [0.0, 0.0, 0.0, 0.0]])
    q, s = quantize_weight_per_channel(w)
    assert torch.equal(s, torch.tensor([1.0, 255.0 / 127.0, 1e-5 / 127.0]))
    assert q.tolist() == [[127, -64, 1, 0], [-127, 127, 1, 0], [0, 0, 0, 0]]   # -63.5 -> -64: half to even
    q, s = quantize_weight_per_channel(w, "torchao")
    eps = torch.finfo(torch.float32).eps
    assert torch.equal(s, torch.tensor([127.0 / 127.5, 2.0, eps]))
    # row 1: +-255 / 2 = +-127.5 -> +-128 (half to even) -> clamped to 127 on the positive side only
    assert q[1].tolist() == [-128, 127, 1, 0]
    assert q[0].tolist() == [127, -64, 1, 0] and q[2].tolist() == [0, 0, 0, 0]   # 127.5 -> 128 -> 127; -63.75 -> -64
    # bf16 weights: the scale is rounded to bf16 and the division runs in bf16, as torch would
    wb = torch.tensor([[3.0, -1.0, 0.5, 0.25]], dtype=torch.bfloat16)
    q, s = quantize_weight_per_channel(wb, "torchao")
    sb = (torch.tensor(3.0) / 127.5).to(torch.bfloat16)
    assert s.dtype == torch.float32 and torch.equal(s, sb.float()[None])
    assert torch.equal(q, torch.round(wb / sb).clamp(-128, 127).to(torch.int8))
    with pytest.raises(ValueError):
        quantize_weight_per_channel(w, "other")


def test_int8_linear_keeps_one_bias():
    """The fp32 bias lives in one buffer; `bias` is a view of it, and loading a float `bias`
    entry (what an nn.Linear state dict carries) lands in that buffer."""
    from samfast_amd import Int8DynamicLinear
    lin = nn.Linear(64, 16)
    q = Int8DynamicLinear.from_float(lin, "torchao")
    assert {k for k in q.state_dict()} == {"sw_bits", "bias_bits", "wq"}
    assert torch.equal(q.bias, lin.bias.detach()) and q.bias.data_ptr() == q.bias_bits.data_ptr()
    sd = q.state_dict()
    del sd["bias_bits"]
    sd["bias"] = torch.full((16,), 0.25, dtype=torch.bfloat16)
    q.load_state_dict(sd)
    assert torch.equal(q.bias_f32, torch.full((16,), 0.25))
    q = q.to(torch.bfloat16)
    assert q.bias.dtype == torch.float32
    assert Int8DynamicLinear.from_float(nn.Linear(64, 16, bias=False)).bias is None
