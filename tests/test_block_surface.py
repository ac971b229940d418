"""Call surface of the block that stands in for the reference's FlashInferBlock (CPU only):
parameter names a reference state dict carries, the attributes the reference's compile
recipe reaches into, batch mode without a cache, and the driver's keyframe rule."""
import pytest
import torch


def make_block(**kw):
    from lingbot_map_amd import HipPagedBlock
    args = dict(dim=128, num_heads=2, mlp_ratio=4.0, qkv_bias=True, proj_bias=True, ffn_bias=True, init_values=0.01,
                qk_norm=True, rope=None, kv_cache_sliding_window=16, kv_cache_scale_frames=1,
                kv_cache_cross_frame_special=True, kv_cache_include_scale_frames=True, kv_cache_camera_only=False)
    args.update(kw)
    return HipPagedBlock(**args)


def test_state_dict_keys_match_reference_block():
    # names from lingbot_map/layers/block.py:183-213 and attention.py:61-67
    expect = {"norm1.weight", "norm1.bias", "attn.qkv.weight", "attn.qkv.bias", "attn.q_norm.weight",
              "attn.q_norm.bias", "attn.k_norm.weight", "attn.k_norm.bias", "attn.proj.weight", "attn.proj.bias",
              "ls1.gamma", "norm2.weight", "norm2.bias", "mlp.fc1.weight", "mlp.fc1.bias", "mlp.fc2.weight",
              "mlp.fc2.bias", "ls2.gamma"}
    assert set(make_block().state_dict().keys()) == expect


def test_attributes_the_compile_recipe_uses():
    b = make_block()
    for name in ("attn_pre", "ffn_residual"):
        assert callable(getattr(b, name))
    assert isinstance(b.attn.proj, torch.nn.Linear)
    assert (b.attn.kv_cache_sliding_window, b.attn.kv_cache_scale_frames) == (16, 1)
    assert b.attn.kv_cache_cross_frame_special and b.attn.kv_cache_include_scale_frames and not b.attn.kv_cache_camera_only


def test_batch_mode_without_cache_is_dense_attention():
    torch.manual_seed(0)
    b = make_block().eval()
    x = torch.randn(2, 11, 128)
    y = b(x)
    # the same arithmetic written out
    h = b.norm1(x)
    q, k, v = b.attn._qkv(h, None, False)
    a = torch.softmax(q @ k.transpose(-1, -2) / 8.0, -1) @ v
    a = b.attn.proj(a.transpose(1, 2).reshape(2, 11, 128))
    ref = b.ffn_residual(x + b.ls1(a))
    assert torch.allclose(y, ref, atol=1e-5)
    q2, k2, v2 = b.attn_pre(x)
    assert q2.shape == (22, 2, 64) and torch.allclose(q2[11:], q[1].permute(1, 0, 2), atol=1e-6)


def test_rotary_matches_complex_multiplication():
    from lingbot_map_amd.block import apply_rotary_emb
    x = torch.randn(1, 2, 5, 8)
    ang = torch.randn(1, 1, 5, 4)
    freqs = torch.polar(torch.ones_like(ang), ang)
    ref = torch.view_as_real(torch.view_as_complex(x.reshape(1, 2, 5, 4, 2)) * freqs).reshape(1, 2, 5, 8)
    assert torch.allclose(apply_rotary_emb(x, freqs), ref, atol=1e-6)


def test_keyframe_flags_follow_driver_rule():
    from lingbot_map_amd import keyframe_flags
    # lingbot_map/models/gct_stream.py:450 with 1 anchor frame and interval 4
    assert keyframe_flags(10, 1, 4) == [True, True, False, False, False, True, False, False, False, True]
    assert sum(keyframe_flags(320, 1, 4)) == 81
    assert all(keyframe_flags(20, 8, 1))


def test_rope2d_module_equals_the_oracle_and_its_table():
    import torch
    from lingbot_map_amd import RotaryPositionEmbedding2D
    from oracle.prepare_qkv import rope2d
    g = torch.Generator().manual_seed(3)
    B, H, N, D = 2, 3, 20, 64
    pos = torch.stack([torch.randint(0, N, (B, N), generator=g), torch.randint(0, N, (B, N), generator=g)], -1)
    rope = RotaryPositionEmbedding2D()
    for dtype in (torch.float32, torch.bfloat16):
        x = torch.randn(B, H, N, D, generator=g).to(dtype)
        assert torch.equal(rope(x, pos), rope2d(x, pos))
        table = rope.cos_sin_table(pos, D, dtype).reshape(B, N, D, 2)
        assert table.dtype == torch.float32
        # x * cos + rotate(x) * sin with the table's values, rounded where torch rounds
        cos, sin = table[..., 0].to(dtype)[:, None], table[..., 1].to(dtype)[:, None]
        rot = torch.cat((-x[..., 16:32], x[..., :16], -x[..., 48:], x[..., 32:48]), -1)
        assert torch.equal(x * cos + rot * sin, rope(x, pos))


def test_rope3d_module_equals_the_oracle_table():
    """The coordinate-based table against the oracle's slice-and-concatenate restatement."""
    from lingbot_map_amd import PositionGetter, RotaryPositionEmbedding3D, WanRotaryPosEmbed
    from oracle.prepare_qkv import rope3d_freqs
    assert WanRotaryPosEmbed is RotaryPositionEmbedding3D
    m = RotaryPositionEmbedding3D(attention_head_dim=64, patch_size=(1, 14, 14), max_seq_len=512)
    assert m.fhw_dim == (20, 22, 22) and not list(m.state_dict())
    for kw in (dict(ppf=1, pph=27, ppw=37, patch_start_idx=6), dict(ppf=3, pph=5, ppw=4, patch_start_idx=6),
               dict(ppf=1, pph=27, ppw=37, patch_start_idx=6, f_start=100, f_end=101),
               dict(ppf=9, pph=3, ppw=7, patch_start_idx=0), dict(ppf=2, pph=2, ppw=2, patch_start_idx=5, f_start=3, f_end=7)):
        got = m(device="cpu", **kw)
        want = rope3d_freqs(head_dim=64, max_seq_len=512, **kw)
        assert got.dtype == want.dtype and got.shape == want.shape
        assert (got - want).abs().max().item() < 1e-13, kw
    auto = RotaryPositionEmbedding3D(attention_head_dim=128, fhw_dim=None)
    assert auto.fhw_dim == (44, 42, 42)
    with pytest.raises(AssertionError):
        m(ppf=1, pph=2, ppw=2, patch_start_idx=0, device="cpu", f_start=511, f_end=513)
    pos = PositionGetter()(2, 3, 4, "cpu")
    assert pos.shape == (2, 12, 2) and pos[1, 7].tolist() == [1, 3] and pos[0, 11].tolist() == [2, 3]


def test_scratch_lanes_nest_and_restore():
    """The lane that keys the package's per-device scratch memory: 0 by default, set for the span
    of a `with`, restored on the way out, also when the body raises."""
    from lingbot_map_amd import _native as N
    assert N.current_scratch_lane() == 0
    with N.scratch_lane(1):
        assert N.current_scratch_lane() == 1
        with N.scratch_lane(2):
            assert N.current_scratch_lane() == 2
        assert N.current_scratch_lane() == 1
    assert N.current_scratch_lane() == 0
    with pytest.raises(ValueError):
        with N.scratch_lane(3):
            raise ValueError("body fails")
    assert N.current_scratch_lane() == 0
