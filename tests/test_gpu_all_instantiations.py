"""Every compiled kernel instantiation is launched at least once and gives the bits of the default one.

The launchers pick among template instantiations (vectors per lane x waves per row x store kind for the
norm, head size x store kind x waves for QKV, unroll x store kind for SwiGLU ...).  The parity tests
pin the defaults against the oracle; this file walks the tuning knobs over shapes chosen so that every
remaining instantiation runs, and requires bit-identical results (the knobs may change speed only).
"""
import itertools

import numpy as np
import pytest
import torch

from helpers import assert_f16_close, assert_f32_close, norm_inputs, qkv_inputs, swiglu_inputs

pytestmark = pytest.mark.gpu
NP2T = {np.float16: torch.float16, np.float32: torch.float32}


def say(msg):
    print("[case] " + msg, flush=True)


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def with_knobs(settings, fn):
    from inferspore_amd import capi
    lib = capi.lib()
    try:
        for knob, value in settings.items():
            assert lib.isp_tuning_set(knob, value) >= 0
        return fn()
    finally:
        for knob in settings:
            lib.isp_tuning_set(knob, 0)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_norm_every_vectors_per_lane_waves_per_row_store_kind_and_workgroup_size(isp, oracle, dtype):
    from inferspore_amd import capi
    vec = 8 if dtype == np.float16 else 4
    for wpr, nv in itertools.product((1, 2, 4, 8, 16), (1, 2, 4, 8)):
        hidden = vec * 64 * wpr * nv - (vec if nv > 1 else 0)  # just inside nv vectors per lane, ragged last vector
        tokens = 7  # not a multiple of the 2, 4 or 8 rows a workgroup carries
        res, out, bias, gamma = norm_inputs(tokens, hidden, dtype, seed=wpr * 10 + nv)
        d_bias, d_gamma = dev(bias), dev(gamma)

        def run():
            d_res, d_out = dev(res), dev(out)
            isp.fused_add_bias_residual_rmsnorm(d_res, d_out, d_bias, d_gamma, 1e-5)
            return d_res.cpu().numpy(), d_out.cpu().numpy()

        base = run()
        e_res, e_out = oracle.fused_norm(res, out, bias, gamma, 1e-5)
        assert np.array_equal(base[0], e_res)
        if dtype == np.float32:
            assert_f32_close(base[1], e_out, "norm hidden %d" % hidden)
        else:
            assert_f16_close(base[1], e_out, "norm hidden %d" % hidden, max_mismatch_fraction=0.05)
        # the row sum is one fixed tree whatever the split of the row over waves and vectors per lane
        # order 1: the default (seven rows take the few-rows kernels where one exists), 2: streaming, 3: the general
        # kernel also for few rows
        for split, store, block, order in itertools.product((1, 2, 4, 8, 16), (1, 2, 3), (256, 512), (1, 2, 3)):  # noqa: E501
            say("norm %s hidden=%d waves/row=%d store=%d block=%d order=%d" % (dtype.__name__, hidden, split, store,
                                                                                 block, order))
            got = with_knobs({capi.TUNE_NORM_WAVES_PER_ROW: split, capi.TUNE_NORM_STORE: store,
                              capi.TUNE_NORM_BLOCK_THREADS: block, capi.TUNE_NORM_ORDER: order}, run)
            assert np.array_equal(got[0], base[0]) and np.array_equal(got[1], base[1])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_norm_few_rows_kernels_match_the_general_kernel_and_the_oracle(isp, oracle, dtype):
    """Launches of a few rows take kernels with the operand set fixed at compile time (one or two vectors per
    lane x waves per row x plain / non-temporal stores x {RMSNorm, residual, residual + bias}); every one of
    them must give the bits of the general kernel (knob order 3) and match the oracle."""
    from inferspore_amd import capi
    lib = capi.lib()
    vec = 8 if dtype == np.float16 else 4
    es = 2 if dtype == np.float16 else 4
    shapes = [(wpr, 1) for wpr in (1, 2, 4, 8, 16)] + [(16, 2)]
    seen = 0
    for (wpr, nv), tokens in itertools.product(shapes, (1, 5)):
        hidden = vec * 64 * wpr * nv - (vec * 3 if wpr * nv > 1 else 0)   # ragged last wave
        for with_res, with_bias in ((False, False), (True, False), (True, True)):
            res, out, bias, gamma = norm_inputs(tokens, hidden, dtype, seed=100 * wpr + 10 * nv + tokens)
            d_bias, d_gamma = (dev(bias) if with_bias else None), dev(gamma)

            def run():
                d_res, d_out = (dev(res) if with_res else None), dev(out)
                if with_res:
                    isp.fused_add_bias_residual_rmsnorm(d_res, d_out, d_bias, d_gamma, 1e-5)
                else:
                    isp.rmsnorm(d_out, d_gamma, 1e-5)
                return (d_res.cpu().numpy() if with_res else None), d_out.cpu().numpy()

            e_res, e_out = oracle.fused_norm(res if with_res else None, out, bias if with_bias else None, gamma, 1e-5)
            general = with_knobs({capi.TUNE_NORM_WAVES_PER_ROW: wpr, capi.TUNE_NORM_ORDER: 3}, run)
            if with_res:
                assert np.array_equal(general[0], e_res)
            if dtype == np.float32:
                assert_f32_close(general[1], e_out, "norm hidden %d" % hidden)
            else:
                assert_f16_close(general[1], e_out, "norm hidden %d" % hidden, max_mismatch_fraction=0.05)
            for store in (1, 2):
                say("few-rows norm %s hidden=%d tokens=%d waves/row=%d residual=%s bias=%s store=%d" % (
                    dtype.__name__, hidden, tokens, wpr, with_res, with_bias, store))
                knobs = {capi.TUNE_NORM_WAVES_PER_ROW: wpr, capi.TUNE_NORM_STORE: store}

                def variant():
                    return lib.isp_norm_launch_variant(es, tokens, hidden, int(with_res), int(with_bias), 0)

                assert with_knobs(knobs, variant) == 1, "this shape must take a few-rows kernel"
                seen += 1
                got = with_knobs(knobs, run)
                if with_res:
                    assert np.array_equal(got[0], general[0])
                assert np.array_equal(got[1], general[1])
    assert seen == len(shapes) * 2 * 3 * 2
    # what the few-rows kernels do not cover goes to the general kernel: the reference's literal residual order,
    # a bias without a residual, more than two vectors per lane, write-through stores, many rows
    assert lib.isp_norm_launch_variant(es, 4, 4096, 1, 1, 1) == 0
    assert lib.isp_norm_launch_variant(es, 4, 4096, 0, 1, 0) == 0
    assert lib.isp_norm_launch_variant(es, 4, vec * 64 * 16 * 4, 1, 0, 0) == 0
    assert lib.isp_norm_launch_variant(es, 16384, 4096, 1, 0, 0) == 0
    assert with_knobs({capi.TUNE_NORM_STORE: 3}, lambda: lib.isp_norm_launch_variant(es, 4, 4096, 1, 0, 0)) == 0


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_norm_pacing_load_gives_the_same_bits(isp, oracle, dtype):
    """A call with a residual and no bias may wait for a gamma vector where the bias vector would arrive (a matter
    of timing only: knob order 5 forces it, 4 forbids it).  Same bits with and without, in every split of the row,
    and the oracle's results at the size where the launcher switches it on by itself."""
    from inferspore_amd import capi
    vec = 8 if dtype == np.float16 else 4
    for wpr, nv in ((1, 1), (2, 2), (4, 4), (8, 8), (16, 2)):
        hidden = vec * 64 * wpr * nv - (vec if nv > 1 else 0)
        # enough rows that the unpaced launch, too, takes the general kernel (the kernels with the operand set
        # fixed at compile time take every launch whose waves are all resident at once, and have no pacing load)
        tokens = 300
        es = 2 if dtype == np.float16 else 4
        unpaced = {capi.TUNE_NORM_WAVES_PER_ROW: wpr, capi.TUNE_NORM_ORDER: 4}
        while with_knobs(unpaced, lambda: capi.lib().isp_norm_launch_variant(es, tokens, hidden, 1, 0, 0)) != 0:
            tokens *= 2
        assert tokens <= 20000
        res, out, _, gamma = norm_inputs(tokens, hidden, dtype, seed=7 * wpr + nv)
        d_gamma = dev(gamma)

        def run():
            d_res, d_out = dev(res), dev(out)
            isp.fused_add_bias_residual_rmsnorm(d_res, d_out, None, d_gamma, 1e-5)
            return d_res.cpu().numpy(), d_out.cpu().numpy()

        e_res, e_out = oracle.fused_norm(res, out, None, gamma, 1e-5)
        for block in (256, 512):
            say("pacing load %s hidden=%d waves/row=%d block=%d" % (dtype.__name__, hidden, wpr, block))
            base = with_knobs({capi.TUNE_NORM_WAVES_PER_ROW: wpr, capi.TUNE_NORM_BLOCK_THREADS: block,
                               capi.TUNE_NORM_ORDER: 4}, run)
            paced = with_knobs({capi.TUNE_NORM_WAVES_PER_ROW: wpr, capi.TUNE_NORM_BLOCK_THREADS: block,
                                capi.TUNE_NORM_ORDER: 5}, run)
            assert np.array_equal(base[0], e_res) and np.array_equal(paced[0], base[0])
            assert np.array_equal(paced[1], base[1])
            if dtype == np.float32:
                assert_f32_close(base[1], e_out, "norm hidden %d" % hidden)
            else:
                assert_f16_close(base[1], e_out, "norm hidden %d" % hidden, max_mismatch_fraction=0.05)
    # 2048 x 4096 with a residual and no bias: the size the default switches the wait on for
    res, out, _, gamma = norm_inputs(2048, 4096, dtype, seed=99)
    d_gamma = dev(gamma)

    def big():
        d_res, d_out = dev(res), dev(out)
        isp.fused_add_bias_residual_rmsnorm(d_res, d_out, None, d_gamma, 1e-5)
        return d_res.cpu().numpy(), d_out.cpu().numpy()

    default = big()
    off = with_knobs({capi.TUNE_NORM_ORDER: 4}, big)
    e_res, e_out = oracle.fused_norm(res, out, None, gamma, 1e-5)
    assert np.array_equal(default[0], e_res) and np.array_equal(default[0], off[0]) and np.array_equal(default[1], off[1])
    if dtype == np.float32:
        assert_f32_close(default[1], e_out, "norm 2048 x 4096 without bias")
    else:
        assert_f16_close(default[1], e_out, "norm 2048 x 4096 without bias", max_mismatch_fraction=0.05)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_norm_rows_do_not_depend_on_the_batch_they_are_in(isp, dtype):
    """The launch configuration changes with the number of rows; a row's result must not."""
    hidden = 4096
    g = torch.Generator(device="cuda").manual_seed(11)
    big_out = torch.randn((9000, hidden), device="cuda", generator=g).to(NP2T[dtype])
    big_res = torch.randn((9000, hidden), device="cuda", generator=g).to(NP2T[dtype])
    gamma = (0.5 + torch.rand(hidden, device="cuda", generator=g)).to(NP2T[dtype])
    ref_out, ref_res = big_out.clone(), big_res.clone()
    isp.fused_add_bias_residual_rmsnorm(ref_res, ref_out, None, gamma, 1e-5)
    ref_plain = big_out.clone()
    isp.rmsnorm(ref_plain, gamma, 1e-5)
    for rows in (1, 3, 64, 700, 2048, 4097):
        say("norm %s: first %d of 9000 rows alone" % (dtype, rows))
        o, r = big_out[:rows].clone(), big_res[:rows].clone()
        isp.fused_add_bias_residual_rmsnorm(r, o, None, gamma, 1e-5)
        assert torch.equal(o, ref_out[:rows]) and torch.equal(r, ref_res[:rows])
        o = big_out[:rows].clone()
        isp.rmsnorm(o, gamma, 1e-5)
        assert torch.equal(o, ref_plain[:rows])


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("hs,hn,kvn", [(64, 16, 8), (128, 12, 4), (128, 32, 32)])
def test_qkv_every_head_size_store_kind_and_wave_count(isp, dtype, hs, hn, kvn):
    from inferspore_amd import capi
    # 64-element heads in whole groups of 8: the automatic choice in fp16 is the two-tokens-per-workgroup
    # kernel, knob 8 the whole-row kernel, 1 / 2 / 4 the general one; 128-element heads in whole groups of 32
    # (fp16) or 16 (fp32): automatic and knob 8 are the one-vector-per-lane kernels, 1 / 2 / 4 the general
    # one -- all must agree to the bit
    batch, seq = 3, 16
    lens, qkv, bias, po, hist = qkv_inputs(batch, seq, hn, kvn, hs, dtype, seed=hs, min_len=2)
    hist = np.array([0, 9, 300], np.int32)
    d_in, d_bias, d_hist, d_lens = dev(qkv), dev(bias), dev(hist), dev(lens)
    po_dev = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
    po_dev.view(-1)[:qkv.shape[0]] = dev(po)

    def run():
        outs = [torch.full((batch, n, seq, hs), -3, dtype=NP2T[dtype], device="cuda") for n in (hn, kvn, kvn)]
        isp.add_fused_qkv_bias_transpose_and_rope(outs[0], outs[1], outs[2], d_in, d_bias, po_dev, d_hist, d_lens,
                                                  hs, 10000.0)
        return [o.cpu().numpy() for o in outs]

    base = run()
    for store, waves in itertools.product((1, 2, 3), (0, 1, 2, 4, 8)):
        say("qkv %s hs=%d store=%d waves=%d" % (dtype.__name__, hs, store, waves))
        got = with_knobs({capi.TUNE_QKV_STORE: store, capi.TUNE_QKV_WAVES: waves}, run)
        assert all(np.array_equal(a, b) for a, b in zip(got, base))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_swiglu_every_unroll_and_store_kind(isp, oracle, dtype):
    from inferspore_amd import capi
    x = swiglu_inputs(21, 11008, dtype, seed=5)
    d_x = dev(x)

    def run():
        out = torch.zeros((21, 11008), dtype=NP2T[dtype], device="cuda")
        isp.act(d_x, out)
        return out.cpu().numpy()

    base = run()
    if dtype == np.float32:
        assert_f32_close(base, oracle.swiglu(x), "swiglu")
    else:
        assert_f16_close(base, oracle.swiglu(x), "swiglu")
    for unroll, store in itertools.product((1, 2, 4), (1, 2, 3)):
        say("swiglu %s unroll=%d store=%d" % (dtype.__name__, unroll, store))
        assert np.array_equal(with_knobs({capi.TUNE_SWIGLU_UNROLL: unroll, capi.TUNE_SWIGLU_STORE: store}, run), base)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_swiglu_vector_and_scalar_kernels_agree_bit_for_bit(isp, dtype):
    """An input at a 16-byte boundary takes the vector kernel, the same values one element further on take
    the scalar one; a caller must not see the difference, in either precision."""
    tokens, inter = 37, 1408
    x = swiglu_inputs(tokens, inter, dtype, seed=17) * dtype(3)
    td = NP2T[dtype]
    aligned_out = torch.zeros((tokens, inter), dtype=td, device="cuda")
    isp.act(dev(x), aligned_out)
    flat = torch.zeros(x.size + 1, dtype=td, device="cuda")
    flat[1:] = dev(x).view(-1)
    shifted_in = flat[1:].view(tokens, 2, inter)
    assert shifted_in.data_ptr() % 16 != 0
    for out_shift in (0, 1):
        say("swiglu %s misaligned input, output shift %d" % (dtype.__name__, out_shift))
        out_flat = torch.zeros(tokens * inter + 1, dtype=td, device="cuda")
        out = out_flat[out_shift:out_shift + tokens * inter].view(tokens, inter)
        isp.act(shifted_in, out)
        assert torch.equal(out, aligned_out)
    say("swiglu %s aligned input, misaligned output" % dtype.__name__)
    out_flat = torch.zeros(tokens * inter + 1, dtype=td, device="cuda")
    out = out_flat[1:].view(tokens, inter)
    isp.act(dev(x), out)
    assert torch.equal(out, aligned_out)


def test_calibration_copy(isp):
    from inferspore_amd import capi
    lib = capi.lib()
    st = torch.cuda.current_stream().cuda_stream
    for nbytes in (16, 4096, (1 << 20) + 16, 48 << 20):
        say("calibration copy of %d bytes" % nbytes)
        src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda")
        dst = torch.zeros(nbytes + 16, dtype=torch.uint8, device="cuda")
        capi.check(lib.isp_calibration_copy(dst.data_ptr(), src.data_ptr(), nbytes, st), "isp_calibration_copy")
        assert torch.equal(dst[:nbytes], src) and int(dst[nbytes:].sum()) == 0


def test_kv_movers_every_workgroup_size(isp):
    from inferspore_amd import capi
    batch, kvn, hn, q_len, max_seq, hs = 3, 2, 4, 70, 96, 128
    g = torch.Generator(device="cuda").manual_seed(3)
    k_src = torch.randn((batch, kvn, q_len, hs), device="cuda", generator=g).half()
    v_src = torch.randn((batch, kvn, q_len, hs), device="cuda", generator=g).half()
    lens = torch.tensor([70, 1, 33], dtype=torch.int32, device="cuda")
    hist = torch.tensor([5, 0, 26], dtype=torch.int32, device="cuda")

    def run():
        kc = torch.full((1, batch, kvn, max_seq, hs), -2.0, dtype=torch.float16, device="cuda")
        vc = kc.clone()
        isp.concat_kv_cache(k_src, v_src, 0, lens, hist, kc, vc)
        kd = torch.full((batch, hn, max_seq, hs), -3.0, dtype=torch.float16, device="cuda")
        vd = kd.clone()
        isp.repeat_kv_cache(kc, vc, lens + hist, 0, kd, vd)
        return [t.cpu().numpy() for t in (kc, vc, kd, vd)]

    base = run()
    # what the four arrays must hold, by plain indexing
    ek = np.full((1, batch, kvn, max_seq, hs), -2.0, np.float16)
    ev = ek.copy()
    ekd = np.full((batch, hn, max_seq, hs), -3.0, np.float16)
    evd = ekd.copy()
    ks, vs = k_src.cpu().numpy(), v_src.cpu().numpy()
    for b, (n, h0) in enumerate(zip(lens.tolist(), hist.tolist())):
        ek[0, b, :, h0:h0 + n] = ks[b, :, :n]
        ev[0, b, :, h0:h0 + n] = vs[b, :, :n]
        for h in range(hn):
            ekd[b, h, :h0 + n] = ek[0, b, h // (hn // kvn), :h0 + n]
            evd[b, h, :h0 + n] = ev[0, b, h // (hn // kvn), :h0 + n]
    assert all(np.array_equal(a, b) for a, b in zip(base, (ek, ev, ekd, evd)))
    for block in (64, 128, 256, 512, 1024):
        say("kv movers with %d-thread workgroups" % block)
        got = with_knobs({capi.TUNE_MOVER_BLOCK_THREADS: block}, run)
        assert all(np.array_equal(a, b) for a, b in zip(got, base))


def test_transpose_out_every_workgroup_size(isp):
    """Single-wave workgroups by default; every compiled workgroup size must move the same bytes, for a row that
    is a whole number of the largest workgroups and for one that is not."""
    from inferspore_amd import capi
    for heads in (32, 40):
        batch, seq, hs = 3, 10, 128
        lens = np.array([10, 3, 7], np.int32)
        tokens = int(lens.sum())
        g = torch.Generator(device="cuda").manual_seed(heads)
        src = torch.randn((batch, heads, seq, hs), device="cuda", generator=g).half()
        po = torch.zeros((batch, seq), dtype=torch.int32, device="cuda")
        po.view(-1)[:tokens] = torch.from_numpy(np.repeat(np.cumsum(seq - lens) - (seq - lens), lens).astype(np.int32)).cuda()

        def run():
            out = torch.full((tokens, heads, hs), -4.0, dtype=torch.float16, device="cuda")
            isp.transpose_out_remove_padding(src, po, out)
            return out.cpu().numpy()

        base = run()
        expect = np.concatenate([src[b, :, :n].permute(1, 0, 2).cpu().numpy() for b, n in enumerate(lens)])
        assert np.array_equal(base, expect)
        for block in (64, 128, 256, 512):
            say("transpose-out, %d heads, %d-thread workgroups" % (heads, block))
            assert np.array_equal(with_knobs({capi.TUNE_MOVER_BLOCK_THREADS: block}, run), base)


def test_kv_movers_more_rows_than_a_grid_dimension_holds(isp):
    """A decode step of a large batch has more (sequence, head) rows than the 65535 a grid's second
    dimension can count; the movers index their workgroups linearly, so it must simply work."""
    batch, kvn, hn, max_seq, hs = 2100, 32, 32, 3, 128
    say("kv movers with %d rows" % (batch * kvn))
    g = torch.Generator(device="cuda").manual_seed(9)
    k_src = torch.randn((batch, kvn, 1, hs), device="cuda", generator=g).half()
    v_src = torch.randn((batch, kvn, 1, hs), device="cuda", generator=g).half()
    lens = torch.ones(batch, dtype=torch.int32, device="cuda")
    hist = (torch.arange(batch, device="cuda") % max_seq).to(torch.int32)
    kc = torch.full((1, batch, kvn, max_seq, hs), -2.0, dtype=torch.float16, device="cuda")
    vc = kc.clone()
    isp.concat_kv_cache(k_src, v_src, 0, lens, hist, kc, vc)
    ek = torch.full_like(kc, -2.0)
    ev = torch.full_like(vc, -2.0)
    rows = torch.arange(batch, device="cuda")
    ek[0, rows, :, hist.long()] = k_src[:, :, 0]
    ev[0, rows, :, hist.long()] = v_src[:, :, 0]
    assert torch.equal(kc, ek) and torch.equal(vc, ev)
    kd = torch.full((batch, hn, max_seq, hs), -3.0, dtype=torch.float16, device="cuda")
    vd = kd.clone()
    isp.repeat_kv_cache(kc, vc, lens + hist, 0, kd, vd)
    live = (torch.arange(max_seq, device="cuda")[None, :] <= hist[:, None].long())[:, None, :, None]
    assert torch.equal(kd, torch.where(live, kc[0], torch.full_like(kd, -3.0)))
    assert torch.equal(vd, torch.where(live, vc[0], torch.full_like(vd, -3.0)))
