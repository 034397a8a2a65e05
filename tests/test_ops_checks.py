"""Host-side extent checks of the torch wrappers: a mis-shaped operand must raise before anything is
launched.  Runs without a GPU -- every case fails its check before the device is touched (a well-shaped
CPU tensor fails the "must live on the GPU" check instead)."""
import pytest
import torch

from inferspore_amd import ops

H = torch.float16
I = torch.int32


def t(*shape, dtype=H):
    return torch.zeros(shape, dtype=dtype)


def test_embedding_checks():
    with pytest.raises(RuntimeError, match="1st shape"):
        ops.input_embedding(t(5, dtype=I), t(4, 8), t(10, 8))
    with pytest.raises(RuntimeError, match="rows"):
        ops.input_embedding(t(4, dtype=I), t(4, 8), t(10, 16))
    with pytest.raises(TypeError):
        ops.input_embedding(t(4, dtype=torch.int64), t(4, 8), t(10, 8))
    with pytest.raises(RuntimeError, match="GPU"):
        ops.input_embedding(t(4, dtype=I), t(4, 8), t(10, 8))


def test_norm_checks():
    with pytest.raises(RuntimeError, match="gamma"):
        ops.rmsnorm(t(4, 8), t(7), 1e-5)
    with pytest.raises(RuntimeError, match="gamma"):
        ops.fused_add_bias_residual_rmsnorm(t(4, 8), t(4, 8), None, t(16), 1e-5)
    with pytest.raises(RuntimeError, match="bias"):
        ops.fused_add_bias_residual_rmsnorm(t(4, 8), t(4, 8), t(9), t(8), 1e-5)
    with pytest.raises(RuntimeError, match="same shape"):
        ops.fused_add_bias_residual_rmsnorm(t(3, 8), t(4, 8), None, t(8), 1e-5)
    x = t(4, 8)
    with pytest.raises(RuntimeError, match="distinct"):
        ops.fused_add_bias_residual_rmsnorm(x, x, None, t(8), 1e-5)
    with pytest.raises(TypeError):
        ops.fused_add_bias_residual_rmsnorm(t(4, 8), t(4, 8), None, t(8, dtype=torch.float32), 1e-5)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.rmsnorm(t(4, 8), t(8), 1e-5)


def _qkv_args(batch=2, seq=4, hn=4, kvn=2, hs=8, tokens=6):
    return dict(q_buf=t(batch, hn, seq, hs), k_buf=t(batch, kvn, seq, hs), v_buf=t(batch, kvn, seq, hs),
                qkv=t(tokens, hn + 2 * kvn, hs), qkv_bias=t((hn + 2 * kvn) * hs),
                padding_offset=t(batch, seq, dtype=I), history_length=t(batch, dtype=I),
                input_length=t(batch, dtype=I), rotary_embedding_dim=hs, rotary_embedding_base=10000.0)


@pytest.mark.parametrize("field,value,match", [
    ("k_buf", t(2, 2, 4, 4), "k_buf"), ("v_buf", t(2, 3, 4, 8), "v_buf"), ("qkv_bias", t(60), "qkv_bias"),
    ("padding_offset", t(5, dtype=I), "padding_offset"), ("history_length", t(1, dtype=I), "history_length"),
    ("input_length", t(1, dtype=I), "input_length"), ("q_buf", t(2, 4, 4, 16), "head size"),
    ("qkv", t(6, 7, 8), "packed head count"),
])
def test_qkv_checks(field, value, match):
    a = _qkv_args()
    a[field] = value
    with pytest.raises(RuntimeError, match=match):
        ops.add_fused_qkv_bias_transpose_and_rope(**a)


def test_qkv_well_shaped_cpu_tensors_reach_the_device_check():
    with pytest.raises(RuntimeError, match="GPU"):
        ops.add_fused_qkv_bias_transpose_and_rope(**_qkv_args())


def test_qkv_append_checks():
    a = _qkv_args()
    a.update(k_cache=t(1, 2, 2, 16, 8), v_cache=t(1, 2, 2, 16, 8), layer_id=0)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.add_fused_qkv_bias_transpose_rope_and_append(**a)
    for bad in (dict(layer_id=1), dict(k_cache=t(1, 2, 3, 16, 8)), dict(v_cache=t(1, 2, 2, 12, 8)),
                dict(k_buf=None)):
        b = dict(a)
        b.update(bad)
        with pytest.raises(RuntimeError):
            ops.add_fused_qkv_bias_transpose_rope_and_append(**b)
    b = dict(a, k_buf=None, v_buf=None)   # both absent is allowed: reaches the device check
    with pytest.raises(RuntimeError, match="GPU"):
        ops.add_fused_qkv_bias_transpose_rope_and_append(**b)


def test_act_checks():
    with pytest.raises(RuntimeError):
        ops.act(t(4, 3, 8), t(4, 8))
    with pytest.raises(RuntimeError, match="output"):
        ops.act(t(4, 2, 8), t(4, 9))
    with pytest.raises(RuntimeError, match="output"):
        ops.act(t(4, 2, 8), t(3, 8))


def test_mover_checks():
    with pytest.raises(RuntimeError, match="packed output"):
        ops.transpose_out_remove_padding(t(2, 4, 4, 8), t(2, 4, dtype=I), t(6, 4, 4))
    with pytest.raises(RuntimeError, match="padding_offset"):
        ops.transpose_out_remove_padding(t(2, 4, 4, 8), t(3, dtype=I), t(6, 4, 8))
    lens = t(2, dtype=I)
    with pytest.raises(RuntimeError, match="caches"):
        ops.concat_kv_cache(t(2, 2, 4, 8), t(2, 2, 4, 8), 0, lens, lens, t(1, 2, 3, 16, 8), t(1, 2, 3, 16, 8))
    with pytest.raises(RuntimeError, match="layer_id"):
        ops.concat_kv_cache(t(2, 2, 4, 8), t(2, 2, 4, 8), 2, lens, lens, t(2, 2, 2, 16, 8), t(2, 2, 2, 16, 8))
    with pytest.raises(RuntimeError, match="length tensors"):
        ops.concat_kv_cache(t(2, 2, 4, 8), t(2, 2, 4, 8), 0, t(1, dtype=I), lens, t(2, 2, 2, 16, 8), t(2, 2, 2, 16, 8))
    with pytest.raises(RuntimeError, match="multiple"):
        ops.repeat_kv_cache(t(1, 2, 3, 16, 8), t(1, 2, 3, 16, 8), lens, 0, t(2, 4, 8, 8), t(2, 4, 8, 8))
    with pytest.raises(RuntimeError, match="batch"):
        ops.repeat_kv_cache(t(1, 3, 2, 16, 8), t(1, 3, 2, 16, 8), lens, 0, t(2, 4, 8, 8), t(2, 4, 8, 8))
    with pytest.raises(RuntimeError, match="caches"):
        ops.rope_decode_and_append(t(2, 8, 8), None, t(1, 2, 3, 16, 8), t(1, 2, 3, 16, 8), 0, lens, 5, 4, 8, 10000.0)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.rope_decode_and_append(t(2, 8, 8), None, t(1, 2, 2, 16, 8), t(1, 2, 2, 16, 8), 0, lens, 5, 4, 8, 10000.0)
