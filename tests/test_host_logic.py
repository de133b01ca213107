"""Host-side mirror of the reference's plug-in surface: registries, runtime patch state, KV-cache
bookkeeping, wrapper construction and the parameter-name contract.  CPU only."""
import pytest
import torch
from torch import nn


def test_layer_registry_picks_most_specific_and_rejects_unknown():
    from hetu_dit_amd.registry import hetuDiTLayerWrappersRegister as R

    class Base(nn.Module):
        pass

    class Child(Base):
        pass

    @R.register(Base)
    class WBase:
        pass

    @R.register(Child)
    class WChild:
        pass

    try:
        assert R.get_wrapper(Base()) is WBase
        assert R.get_wrapper(Child()) is WChild
        with pytest.raises(ValueError, match="is not supported by hetuDiT"):
            R.get_wrapper(nn.Identity())
    finally:
        R._HETUDIT_LAYER_MAPPING.pop(Base)
        R._HETUDIT_LAYER_MAPPING.pop(Child)


def test_processor_registry_requires_subclass_and_returns_class():
    from hetu_dit_amd.layers import attention_processor as ap
    from hetu_dit_amd.layers.modules import FluxAttnProcessor2_0, JointAttnProcessor2_0
    from hetu_dit_amd.registry import hetuDiTAttentionProcessorRegister as R

    assert R.get_processor(JointAttnProcessor2_0()) is ap.hetuDiTJointAttnProcessor2_0
    assert R.get_processor(FluxAttnProcessor2_0()) is ap.hetuDiTFluxAttnProcessor2_0
    with pytest.raises(ValueError):
        R.get_processor(object())
    with pytest.raises(ValueError):
        @R.register(JointAttnProcessor2_0)
        class NotASubclass:
            pass


def test_runtime_state_patches_match_reference_arithmetic():
    from hetu_dit_amd.runtime_state import DiTRuntimeState

    rs = DiTRuntimeState()
    rs.set_patches(latents_height=128, latents_width=128, patch_size=2, num_pipeline_patch=4)
    assert rs.num_pipeline_patch == 4
    assert rs.pp_patches_height == [32, 32, 32, 32]
    assert rs.pp_patches_token_start_idx_local == [0, 1024, 2048, 3072, 4096]
    # uneven: 100 rows / 3 patches -> heights rounded up to a multiple of the patch size
    rs.set_patches(latents_height=100, latents_width=64, patch_size=2, num_pipeline_patch=3)
    assert rs.pp_patches_height == [34, 34, 32]
    assert rs.pp_patches_token_start_idx_local == [0, 32 * 17, 32 * 34, 32 * 50]
    rs.set_patched_mode(True)
    seen = []
    for _ in range(7):
        seen.append(rs.pipeline_patch_idx)
        rs.next_patch()
    assert seen == [0, 1, 2, 0, 1, 2, 0]
    rs.set_patched_mode(False)
    rs.next_patch()
    assert rs.pipeline_patch_idx == 0


def test_cache_manager_registration_and_patch_range():
    from hetu_dit_amd.cache_manager import CacheManager
    from hetu_dit_amd.runtime_state import get_runtime_state, reset_runtime_state

    rs = reset_runtime_state()
    cm = CacheManager()
    layer = object()
    with pytest.raises(ValueError, match="Layer type"):
        cm.register_cache_entry(layer, "mlp")
    with pytest.raises(ValueError, match="Cache type"):
        cm.register_cache_entry(layer, "attn", "lru")
    cm.register_cache_entry(layer, "attn", "naive_cache")
    assert cm._patch_range() is None  # patch mode off
    rs.set_token_patches([0, 64, 128])
    assert cm._patch_range() is None  # still off
    rs.set_patched_mode(True)
    assert cm._patch_range() == (0, 64)
    rs.next_patch()
    assert cm._patch_range() == (64, 128)
    with pytest.raises(RuntimeError, match="before a full-sequence pass"):
        cm.kv_buffer(layer, 1, 64, 8, "cpu")
    with pytest.raises(KeyError):
        cm._entry(object(), "attn")
    reset_runtime_state()


def test_wrappers_rehome_biases_and_keep_parameter_paths():
    from hetu_dit_amd import blocks
    from hetu_dit_amd.cache_manager import reset_cache_manager

    blk = blocks.JointTransformerBlock(128, 2, 64)
    names = {n for n, _ in blk.named_parameters()}
    for n in ("attn.module.to_q.weight", "attn.module.add_k_proj.bias", "attn.module.to_out.0.weight",
              "attn.module.to_add_out.weight", "attn.output_bias", "attn.encoder_output_bias",
              "ff.module.net.0.proj.weight", "ff.module.net.2.weight", "ff.output_bias",
              "ff_context.module.net.0.proj.bias", "norm1.linear.weight", "norm1_context.linear.bias"):
        assert n in names, n
    assert "attn.module.to_out.0.bias" not in names and "ff.module.net.2.bias" not in names
    assert blk.attn.has_output_bias and blk.attn.has_encoder_output_bias and blk.ff.has_output_bias
    # attribute fall-through to the wrapped module
    assert blk.attn.heads == 2 and blk.attn.to_q is blk.attn.module.to_q
    last = blocks.JointTransformerBlock(128, 2, 64, context_pre_only=True)
    assert last.ff_context is None and not hasattr(last.attn.module, "to_add_out")
    assert last.norm1_context.linear.weight.shape == (256, 128)
    cog = blocks.CogVideoXBlock(128, 2, 64, time_embed_dim=32)
    assert "attn1.module.norm_q.bias" in {n for n, _ in cog.named_parameters()}
    reset_cache_manager()


def test_packed_projection_views_and_repack():
    from hetu_dit_amd.layers.attention_processor import _PackedProjection

    a, b, c = nn.Linear(8, 4), nn.Linear(8, 4), nn.Linear(8, 6)
    pk = _PackedProjection([a, b, c])
    w, bias = pk.get()
    assert w.shape == (14, 8) and bias.shape == (14,)
    assert a.weight.data_ptr() == w.data_ptr() and c.weight.data_ptr() == w[8:].data_ptr()
    w[0, 0] = 42.0
    assert a.weight[0, 0].item() == 42.0  # the Linear is a view of the packed buffer
    # weight hot-swap re-assigns .data: the pack must notice and rebuild
    b.weight.data = torch.full((4, 8), 7.0)
    w2, _ = pk.get()
    assert w2.data_ptr() != w.data_ptr() and torch.all(w2[4:8] == 7.0)
    wq, bq = pk.rows(4, 4)
    assert torch.all(wq == 7.0) and bq.shape == (4,)
    # a bias alone re-assigned: the packed bias must follow
    c.bias.data = torch.full((6,), 3.0)
    _, b3 = pk.get()
    assert torch.all(b3[8:] == 3.0) and c.bias.data_ptr() == b3[8:].data_ptr()
    with pytest.raises(ValueError, match="all have a bias"):
        _PackedProjection([nn.Linear(8, 4), nn.Linear(8, 4, bias=False)])


def test_wrap_layers_and_register_cache_follow_the_reference_rules():
    """``_wrap_layers`` + ``_register_cache`` of the reference (models/base_model.py:59-112,:162-178) on the
    stand-in classes: children are wrapped by *name* ("attn") or by *class* (FeedForward), constructed through
    the registry, and the K/V cache entry is keyed by the attention *wrapper* -- the object the processors
    later pass as ``layer=attn``."""
    from hetu_dit_amd.base_model import register_cache, wrap_layers
    from hetu_dit_amd.cache_manager import get_cache_manager, reset_cache_manager
    from hetu_dit_amd.layers.attention_processor import hetuDiTAttentionWrapper, hetuDiTJointAttnProcessor2_0
    from hetu_dit_amd.layers.feedforward import hetuDiTFeedForwardWrapper
    from hetu_dit_amd.layers.modules import Attention, FeedForward, JointAttnProcessor2_0

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = Attention(64, 2, 32, added_kv_proj_dim=64, context_pre_only=False, bias=True,
                                  processor=JointAttnProcessor2_0())
            self.ff = FeedForward(64)
            self.other = nn.Linear(64, 64)

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.transformer_blocks = nn.ModuleList([Block(), Block()])

    reset_cache_manager()
    model = Model()
    raw_attn = model.transformer_blocks[0].attn
    wrapped = wrap_layers(model, submodule_classes_to_wrap=[FeedForward], submodule_name_to_wrap=["attn"])
    assert len(wrapped) == 4
    blk = model.transformer_blocks[0]
    assert isinstance(blk.attn, hetuDiTAttentionWrapper) and blk.attn.module is raw_attn
    assert isinstance(blk.ff, hetuDiTFeedForwardWrapper) and isinstance(blk.other, nn.Linear)
    assert isinstance(blk.attn.processor, hetuDiTJointAttnProcessor2_0)
    # parameter paths gain the .module hop; re-homed biases live on the wrapper
    names = dict(model.named_parameters())
    assert "transformer_blocks.0.attn.module.to_q.weight" in names
    assert "transformer_blocks.0.attn.output_bias" in names and "transformer_blocks.1.ff.output_bias" in names
    cm = get_cache_manager()
    assert not cm.cache
    register_cache(wrapped)
    assert set(cm.cache) == {("attn", b.attn) for b in model.transformer_blocks}
    cm._entry(blk.attn, "attn")  # the wrapper is the key
    with pytest.raises(KeyError):
        cm._entry(blk.attn.module, "attn")
    # wrapping again leaves wrappers alone
    assert wrap_layers(model, [FeedForward], ["attn"]) == []
    reset_cache_manager()


def test_wrap_layers_with_the_reference_sd3_class_list():
    """The reference wraps the SD3 transformer with ``submodule_classes_to_wrap=[FeedForward, nn.Conv2d,
    PatchEmbed]``, ``submodule_name_to_wrap=["attn"]`` (models/transformers/transformer_sd3.py:36).  The walk
    skips a wrapper but goes on into the module it wraps, so the patch embedding's ``proj`` gets the Conv2d
    wrapper (layers/conv.py:19-31) and the patch-embedding wrapper must still find ``proj.weight`` / ``.bias``
    through it."""
    from hetu_dit_amd.base_model import wrap_layers
    from hetu_dit_amd.layers.conv import hetuDiTConv2dWrapper
    from hetu_dit_amd.layers.embeddings import hetuDiTPatchEmbedWrapper
    from hetu_dit_amd.layers.modules import FeedForward, PatchEmbed
    from hetu_dit_amd.registry import hetuDiTLayerWrappersRegister
    from hetu_dit_amd.transformer_sd3 import SD3Transformer2DModel

    assert hetuDiTLayerWrappersRegister.get_wrapper(nn.Conv2d(3, 4, 2, 2)) is hetuDiTConv2dWrapper
    model = SD3Transformer2DModel(sample_size=16, num_layers=2, attention_head_dim=64, num_attention_heads=2,
                                  joint_attention_dim=64, caption_projection_dim=128, pooled_projection_dim=64,
                                  pos_embed_max_size=16)
    conv = model.pos_embed.module.proj
    wrapped = wrap_layers(model, [FeedForward, nn.Conv2d, PatchEmbed], ["attn"])
    assert len(wrapped) == 1 and wrapped[0] is model.pos_embed.module.proj
    w = model.pos_embed.module.proj
    assert isinstance(w, hetuDiTConv2dWrapper) and w.module is conv and w.is_first_layer
    assert isinstance(model.pos_embed, hetuDiTPatchEmbedWrapper)
    # attribute fall-through: what the patch-embedding wrapper reads
    assert model.pos_embed.module.proj.weight is conv.weight and model.pos_embed.module.proj.bias is conv.bias
    assert "pos_embed.module.proj.module.weight" in dict(model.named_parameters())
    # an unwrapped model gets the same result from the same call: PatchEmbed first, then its proj
    class Bare(nn.Module):
        def __init__(self):
            super().__init__()
            self.pos_embed = PatchEmbed(16, 16, 2, 4, 64, pos_embed_max_size=8)

    bare = Bare()
    wrapped = wrap_layers(bare, [FeedForward, nn.Conv2d, PatchEmbed], ["attn"])
    assert [type(x) for x in wrapped] == [hetuDiTPatchEmbedWrapper, hetuDiTConv2dWrapper]
    assert isinstance(bare.pos_embed.module.proj, hetuDiTConv2dWrapper)
    # geometry the wrapper does not run is refused, not handed to a library convolution
    odd = hetuDiTConv2dWrapper(nn.Conv2d(4, 8, 3, stride=1, padding=1), is_first_layer=False)
    with pytest.raises(NotImplementedError, match="kernel = stride"):
        odd._patch_size()


def test_patch_embed_height_from_input_config():
    """The patch-embedding wrapper takes the whole image's latent rows from input_config.height //
    vae_scale_factor like the reference (layers/embeddings.py:33-36), else from set_patches."""
    from hetu_dit_amd.runtime_state import reset_runtime_state

    rs = reset_runtime_state()
    assert rs.whole_image_latent_rows() == 0
    rs.set_patches(latents_height=128, latents_width=128, patch_size=2, num_pipeline_patch=4)
    assert rs.whole_image_latent_rows() == 128
    rs.set_input_parameters(height=512, width=512, vae_scale_factor=8)
    assert rs.whole_image_latent_rows() == 64
    reset_runtime_state()


def test_ops_refuse_cpu_tensors():
    from hetu_dit_amd import ops

    x = torch.zeros(1, 4, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.layernorm_modulate(x)
    with pytest.raises(ValueError, match="no CPU path"):
        ops.linear(x, torch.zeros(64, 64, dtype=torch.bfloat16))


def test_single_rank_parallel_state():
    from hetu_dit_amd import parallel_state as ps

    assert ps.get_tensor_model_parallel_world_size() == 1 and ps.get_sequence_parallel_world_size() == 1
    assert ps.get_pipeline_parallel_world_size() == 1 and ps.is_pipeline_first_stage() and ps.is_pipeline_last_stage()
    t = torch.ones(2)
    assert ps.get_tp_group().all_reduce(t) is t


def test_torch_library_ops_have_fake_kernels():
    """torch.ops.hdit.* trace under FakeTensorMode without touching a device."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    import hetu_dit_amd.torch_ops  # noqa: F401

    with FakeTensorMode():
        x = torch.empty(2, 7, 64, dtype=torch.bfloat16, device="cuda")
        w = torch.empty(128, 64, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.hdit.linear(x, w).shape == (2, 7, 128)
        assert torch.ops.hdit.layernorm_modulate(x).shape == x.shape
        t = torch.empty(2, 64, dtype=torch.bfloat16, device="cuda")
        out = torch.ops.hdit.adaln_gemv(t, w)
        assert out.shape == (2, 128) and out.dtype == torch.float32
        q = torch.empty(2, 7, 1, 64, dtype=torch.bfloat16, device="cuda")
        (o,) = torch.ops.hdit.attention([q], [q], [q])
        assert o.shape == q.shape
        lat = torch.empty(2, 16, 8, 12, dtype=torch.bfloat16, device="cuda")
        tok = torch.ops.hdit.patchify(lat, 2)
        assert tok.shape == (2, 24, 64)
        assert torch.ops.hdit.unpatchify(tok, 16, 8, 12, 2).shape == lat.shape
        ts = torch.empty(3, dtype=torch.float32, device="cuda")
        emb = torch.ops.hdit.timestep_embedding(ts, 256)
        assert emb.shape == (3, 256) and emb.dtype == torch.bfloat16
        assert torch.ops.hdit.silu(emb).shape == emb.shape
        cos, sin = torch.ops.hdit.rope_table(torch.empty(9, 3, dtype=torch.float32, device="cuda"), [16, 56, 56])
        assert cos.shape == sin.shape == (9, 128) and cos.dtype == torch.float32
        assert torch.ops.hdit.cfg_euler_step(lat, lat, lat, 7.0, 1.0, 0.9).shape == lat.shape


def test_feed_forward_wrapper_recognises_foreign_first_layers_and_slices_geglu_per_half(monkeypatch):
    """The wrapper reads a first layer by class name as well as by class (an instance of diffusers' own ``GELU`` /
    ``GEGLU`` / ``LinearActivation`` is not an instance of the classes here), takes diffusers' ``approximate="none"``
    default, slices the value and gate halves of a GEGLU projection separately per tensor-parallel rank
    (reference ``layers/feedforward.py:34-46``) and refuses what it has no kernel for."""
    from hetu_dit_amd import ops
    from hetu_dit_amd.layers import feedforward as ffmod
    from hetu_dit_amd.layers.feedforward import hetuDiTFeedForwardWrapper

    def foreign(name, width, **attrs):
        cls = type(name, (nn.Module,), {})
        m = cls()
        m.proj = nn.Linear(8, width)
        for k, v in attrs.items():
            setattr(m, k, v)
        return m

    def ff_with(first, inner):
        ff = nn.Module()
        ff.net = nn.ModuleList([first, nn.Dropout(0.0), nn.Linear(inner, 8)])
        return ff

    assert hetuDiTFeedForwardWrapper(ff_with(foreign("GELU", 16, approximate="tanh"), 16)).activation_kind is None
    assert hetuDiTFeedForwardWrapper(ff_with(foreign("GELU", 16, approximate="none"), 16)).activation_kind == ops.ACT_GELU_ERF
    assert hetuDiTFeedForwardWrapper(ff_with(foreign("GELU", 16), 16)).activation_kind == ops.ACT_GELU_ERF
    assert hetuDiTFeedForwardWrapper(ff_with(foreign("GEGLU", 32), 16)).activation_kind == ops.ACT_GEGLU
    assert hetuDiTFeedForwardWrapper(ff_with(foreign("LinearActivation", 16, activation=nn.SiLU()), 16)).activation_kind == ops.ACT_SILU
    with pytest.raises(TypeError):
        hetuDiTFeedForwardWrapper(ff_with(foreign("LinearActivation", 16, activation=nn.ReLU()), 16))
    with pytest.raises(TypeError):
        hetuDiTFeedForwardWrapper(ff_with(foreign("SwiGLU", 32), 16))
    with pytest.raises(TypeError):
        hetuDiTFeedForwardWrapper(ff_with(foreign("GELU", 16, approximate="sigmoid"), 16))

    # rank 1 of 2: rows [4, 8) of the value half followed by rows [4, 8) of the gate half; net[2] keeps columns [4, 8)
    monkeypatch.setattr(ffmod, "get_tensor_model_parallel_world_size", lambda: 2)
    monkeypatch.setattr(ffmod, "get_tensor_model_parallel_rank", lambda: 1)
    first = foreign("GEGLU", 16)
    w, b = first.proj.weight.data.clone(), first.proj.bias.data.clone()
    ff = ff_with(first, 8)
    w2 = ff.net[2].weight.data.clone()
    wrapped = hetuDiTFeedForwardWrapper(ff)
    assert torch.equal(wrapped.module.net[0].proj.weight.data, torch.cat([w[4:8], w[12:16]]))
    assert torch.equal(wrapped.module.net[0].proj.bias.data, torch.cat([b[4:8], b[12:16]]))
    assert torch.equal(wrapped.module.net[2].weight.data, w2[:, 4:8])
    assert wrapped.has_output_bias and wrapped.module.net[2].bias is None
