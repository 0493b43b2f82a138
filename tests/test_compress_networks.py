"""Alternative compression networks (compress_networks.py:19-241): each checked on the CPU
against an independent formulation - the einops mixing layer the reference builds them from
(a library routine, loaded with the same parameters), a per-window loop, or a closed form."""
import torch

from native_sparse_attention_pytorch_amd import compress_networks as CN


def test_headwise_linear_matches_einops_mix_layer():
    from einops.layers.torch import EinMix
    torch.manual_seed(0)
    mine = CN.HeadwiseLinear(3, 10, 7)
    lib = EinMix('b h w i -> b h w o', weight_shape='h i o', bias_shape='h o', h=3, i=10, o=7)
    assert {k: v.shape for k, v in mine.state_dict().items()} == {k: v.shape for k, v in lib.state_dict().items()}
    lib.load_state_dict(mine.state_dict())
    x = torch.randn(2, 3, 5, 10)
    assert torch.allclose(mine(x), lib(x), atol=1e-5)
    # initialisation bounds of the mixing layer
    assert mine.weight.abs().max() <= (3 / 10) ** 0.5 and mine.bias.abs().max() <= (1 / 10) ** 0.5


def test_grouped_mlp_matches_per_head_loop_and_reference_parameter_names():
    torch.manual_seed(1)
    m = CN.GroupedMLP(dim_head=8, compress_window_size=4, heads=3, expand_factor=0.5)
    assert set(m.state_dict()) == {"net.0.weight", "net.0.bias", "net.2.weight", "net.2.bias"}
    assert m.net[0].weight.shape == (3, 32, 16) and m.net[2].weight.shape == (3, 16, 8)
    kv = torch.randn(2, 3, 5, 4, 8)
    out = m(kv)
    assert out.shape == (2, 3, 5, 8)
    for h in range(3):
        x = kv[:, h].flatten(-2)
        hid = torch.relu(x @ m.net[0].weight[h] + m.net[0].bias[0, h, 0])
        assert torch.allclose(out[:, h], hid @ m.net[2].weight[h] + m.net[2].bias[0, h, 0], atol=1e-5)


def test_single_projection_both_forms():
    torch.manual_seed(2)
    kv = torch.randn(2, 3, 5, 4, 8)
    shared = CN.SingleProjection(8, 4)
    assert set(shared.state_dict()) == {"compress.1.weight"}
    assert torch.allclose(shared(kv), kv.flatten(-2) @ shared.compress[1].weight.t(), atol=1e-5)
    grouped = CN.SingleProjection(8, 4, heads=3)
    assert set(grouped.state_dict()) == {"compress.weight"}
    want = torch.einsum('bhwni,hio->bhwo', kv, grouped.compress.weight)          # tokens of the window are summed
    assert torch.allclose(grouped(kv), want, atol=1e-4)


def test_conv_compress_is_a_per_head_linear_map_of_each_window():
    torch.manual_seed(3)
    m = CN.ConvLinearCompress(heads=3, dim_head=4, compress_window_size=5)
    kv = torch.randn(2, 3, 6, 5, 4)
    out = m(kv)
    assert out.shape == (2, 3, 6, 4)
    wgt = m.conv.weight.view(3, 4, 4, 5)                                       # head, out feature, in feature, token
    want = torch.einsum('bhwni,hoin->bhwo', kv, wgt) + m.conv.bias.view(3, 4)[None, :, None]
    assert torch.allclose(out, want, atol=1e-5)


def test_attention_pool_identity_init_and_mean_limit():
    m = CN.AttentionPool(8, 4)
    kv = torch.randn(2, 3, 5, 4, 8)
    assert torch.allclose(m(kv), (kv * kv.softmax(dim=-2)).sum(dim=-2), atol=1e-6)
    with torch.no_grad():
        m.to_attn_logits.weight.zero_()
    assert torch.allclose(m(kv), kv.mean(dim=-2), atol=1e-6)


def test_compress_transformer_shapes_and_last_token_semantics():
    torch.manual_seed(4)
    m = CN.CompressTransformer(num_layers=2, dim=3 * 8, num_heads=2)
    names = set(m.state_dict())
    assert "layers.1.attn.q_proj.weight" in names and "layers.0.ff.fc2.bias" in names and "layers.1.norm2.weight" in names
    kv = torch.randn(2, 3, 5, 4, 8)
    out = m(kv)
    assert out.shape == (2, 3, 5, 8)
    # equals running both full layers and taking the last token (the feed-forward is per token)
    t = kv.permute(0, 2, 3, 1, 4).reshape(10, 4, 24)
    for layer in m.layers:
        t = layer(t)
    assert torch.allclose(out, t[:, -1].reshape(2, 5, 3, 8).permute(0, 2, 1, 3), atol=1e-5)
    # windows are independent
    kv2 = kv.clone()
    kv2[:, :, 2] += 1.0
    out2 = m(kv2)
    assert torch.allclose(out[:, :, [0, 1, 3, 4]], out2[:, :, [0, 1, 3, 4]], atol=1e-6)
    assert not torch.allclose(out[:, :, 2], out2[:, :, 2])


def test_oracle_module_accepts_the_networks_and_decode_still_equals_parallel():
    """The networks plugged into the (CPU) oracle module: token-by-token decode reproduces the
    parallel forward, i.e. window handling is consistent for every network."""
    from oracle import nsa_oracle as O
    for mk in (lambda: CN.GroupedMLP(16, 4, 2), lambda: CN.ConvLinearCompress(2, 16, 4), lambda: CN.AttentionPool(16, 4),
               lambda: CN.SingleProjection(16, 4, heads=2), lambda: CN.CompressTransformer(1, 32, 2)):
        torch.manual_seed(5)
        m = O.SparseAttentionOracle(dim=32, dim_head=16, heads=4, kv_heads=2, causal=True, sliding_window_size=3, compress_block_size=4,
                                    compress_block_sliding_stride=2, selection_block_size=4, num_selected_blocks=2, compress_mlp=mk())
        x = torch.randn(1, 19, 32)
        par = m(x)
        cache, outs = None, []
        for i in range(19):
            o, cache = m(x[:, i:i + 1], cache=cache, return_cache=True)
            outs.append(o)
        assert torch.allclose(par, torch.cat(outs, dim=1), atol=1e-5)
