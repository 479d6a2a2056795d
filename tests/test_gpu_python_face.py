"""The Python face over torch tensors: a LoRA-shaped training loop against the oracle."""
import numpy as np
import pytest
import torch

import harness as hs
import oracle_c as oc
from oracle import adam8_numpy as onp

pytestmark = pytest.mark.gpu


def _bf16_tensor(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()


def _bits(t):
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16)


def test_adam8bit_over_torch_parameters_matches_the_oracle(tmp_path):
    from eridiffusion_amd.adam8bit import Adam8bit, Adam8bitConfig, create_optimizer
    sizes = [16 * 640, 1280 * 16, 300]
    ps, _ = hs.make_inputs(sizes, True, 5, p_std=1e-2)
    states = hs.oracle_states(sizes)
    params = [_bf16_tensor(p) for p in ps]
    opt = Adam8bit(params, Adam8bitConfig(lr=1e-3), flags=2)
    for t in (1, 2, 3):
        gs = hs.fresh_grads(sizes, True, 100 + t, 1e-3)
        for p, g in zip(params, gs):
            p.grad = _bf16_tensor(g)
        assert opt.step() == 0
        hs.oracle_step(ps, gs, states, (1e-3, 0.9, 0.999, 1e-8, 0.01, t), True)
        opt.zero_grad()
    torch.cuda.synchronize()
    for p, want in zip(params, ps):
        assert np.array_equal(_bits(p), want)
    assert opt.get_step() == 3 and opt.current_lr() == 1e-3
    assert opt.quantized_memory_usage() == sum(2 * n + 8 * ((n + 2047) // 2048) for n in sizes)
    assert opt.step() == 3  # no gradients left: every parameter skipped, nothing launched
    opt.save_state(tmp_path / "opt.safetensors")
    again = create_optimizer("adamw8bit", params, learning_rate=1e-3)
    again.load_state(tmp_path / "opt.safetensors")
    assert again.get_step() == 4
    with pytest.raises(ValueError, match="Unknown optimizer"):
        create_optimizer("lion", params)


def test_functional_flavour_over_torch_tensors():
    from eridiffusion_amd.adam8bit import Adam8bitFunctional, update_params_8bit
    n = 2048 * 2 + 9
    ps, gs = hs.make_inputs([n], False, 9)
    states = hs.oracle_states([n])
    opt = Adam8bitFunctional.with_params(1e-4, 0.9, 0.999, 1e-8, 0.01)
    params = {"blk.lora_up": torch.from_numpy(ps[0].copy()).cuda(), "frozen": torch.ones(8, device="cuda")}
    grads = {"blk.lora_up": torch.from_numpy(gs[0].copy()).cuda()}
    before = params["blk.lora_up"]
    update_params_8bit(opt, params, grads)
    opt.step()
    hs.oracle_step(ps, gs, states, (1e-4, 0.9, 0.999, 1e-8, 0.01, 0), False, mode=oc.MODE_L2)
    torch.cuda.synchronize()
    assert params["blk.lora_up"] is not before and np.array_equal(before.cpu().numpy(), hs.make_inputs([n], False, 9)[0][0])
    assert np.array_equal(params["blk.lora_up"].cpu().numpy().view(np.uint32), ps[0].view(np.uint32))
    assert opt.get_step() == 1 and opt.memory_stats() == (1, 2 * n + 8 * 3)
    st = opt.get_state_as_tensors()
    m, v = st["blk.lora_up"]
    want_m = hs.MAPS[0][states[0][0]] * np.repeat(states[0][2], 2048)[:n]
    assert np.array_equal(m.cpu().numpy(), want_m.astype(np.float32))
    fresh = Adam8bitFunctional()
    fresh.load_state_from_tensors(st)
    assert fresh.memory_stats() == (1, 2 * n + 8 * 3)
    m2, _ = fresh.get_state_as_tensors()["blk.lora_up"]
    # re-quantising exported moments loses at most half a map step of the (possibly smaller) new absmax
    m_np, m2_np = m.cpu().numpy(), m2.cpu().numpy()
    step = np.diff(hs.MAPS[0]).max() / 2 * np.repeat(states[0][2], 2048)[:n]
    assert np.all(np.abs(m2_np - m_np) <= step * 1.0001)


def test_mode_bnb_with_clipping_and_statistics_through_the_python_face():
    """set_mode(MODE_BNB), clipping inside step() and the error statistics, against the oracle."""
    from eridiffusion_amd import _lib as L
    from eridiffusion_amd.adam8bit import Adam8bit, Adam8bitConfig
    sizes = [2048 * 3 + 17, 640]
    ps, _ = hs.make_inputs(sizes, True, 15, p_std=1e-2)
    states = hs.oracle_states(sizes)
    params = [_bf16_tensor(p) for p in ps]
    opt = Adam8bit(params, Adam8bitConfig(lr=1e-3), flags=L.FLAG_EXACT_PARAM)  # bit-for-bit bf16 parameters
    opt.set_mode(L.MODE_BNB)
    opt.set_max_grad_norm(0.05)
    opt.track_quantization_error(True)
    with pytest.raises(L.EriError):
        opt.set_mode(L.MODE_L2)
    for t in (1, 2):
        gs = hs.fresh_grads(sizes, True, 200 + t, 1e-3)
        for p, g in zip(params, gs):
            p.grad = _bf16_tensor(g)
        assert opt.step() == 0
        norm, scale = opt.last_grad_norm()
        assert norm > 0.05 and scale == np.float32(0.05) / np.float32(norm)
        assert opt.last_nonfinite_grads() == 0
        hs.oracle_step(ps, gs, states, (1e-3, 0.9, 0.999, 1e-8, 0.01, t), True, mode=oc.MODE_BNB,
                       grad_scale=float(np.float32(1.0) * np.float32(scale)))
    torch.cuda.synchronize()
    for p, want in zip(params, ps):
        assert np.array_equal(_bits(p), want)
    m_err, v_err = opt.quantization_stats()
    assert 0 < m_err < 1e-4 and 0 < v_err < 1e-6


def test_ema_model_as_in_the_reference_and_against_the_oracle():
    """ema_enhanced.rs:296-318 restated (decay 0.999, one parameter of 10 fp32 values: init, one update,
    step() == 1, the shadow is there), then the numbers: three updates of two parameters with the
    effective decay of each step, a late-comer adopted by copy, and copy_to."""
    from eridiffusion_amd import _lib as L
    from eridiffusion_amd.adam8bit import EMAModel
    ema = EMAModel(0.999)
    param1 = torch.randn(10, device="cuda")
    ema.init_from_params({"param1": param1})
    ema.update({"param1": param1})
    assert ema.step() == 1 and "param1" in ema and "other" not in ema

    rng = np.random.default_rng(3)
    ema = EMAModel(0.99, use_bias_correction=True, power=1.0)
    w32 = rng.standard_normal(2048 * 2 + 77).astype(np.float32)
    b16 = onp.f32_to_bf16(rng.standard_normal(640).astype(np.float32))
    tw, tb = torch.from_numpy(w32.copy()).cuda(), _bf16_tensor(b16)
    params = {"w": tw, "b": tb}
    ema.init_from_params(params)
    sh_w, sh_b = w32.copy(), b16.copy()
    for step in (1, 2, 3):
        w32 = (w32 + rng.standard_normal(w32.size).astype(np.float32) * np.float32(0.1)).astype(np.float32)
        b16 = onp.f32_to_bf16(onp.bf16_to_f32(b16) + rng.standard_normal(b16.size).astype(np.float32) * np.float32(0.1))
        tw.copy_(torch.from_numpy(w32))
        tb.copy_(_bf16_tensor(b16))
        if step == 3:
            late = torch.full((33,), 2.5, device="cuda")
            params["late"] = late
        ema.update(params)
        d = L.lib().eri_ema_effective_decay(0.99, step, 1.0, 1)
        assert ema.current_decay() == d and ema.step() == step
        oc.lib().eri_oracle_ema_update(oc.ptr(sh_w), oc.ptr(w32), w32.size, oc.DT_F32, d)
        oc.lib().eri_oracle_ema_update(oc.ptr(sh_b), oc.ptr(b16), b16.size, oc.DT_BF16, d)
    got = ema.shadow_params(params)
    torch.cuda.synchronize()
    assert np.array_equal(got["w"].cpu().numpy().view(np.uint32), sh_w.view(np.uint32))
    assert np.array_equal(_bits(got["b"]), sh_b)
    assert bool((got["late"] == 2.5).all())  # first seen at step 3: adopted as a copy
    # the first step's effective decay is 0 (bias correction), so the shadow jumps to the parameter there
    assert L.lib().eri_ema_effective_decay(0.99, 1, 1.0, 1) == 0.0
    target = {"w": torch.zeros_like(tw), "b": torch.zeros_like(tb)}
    ema.copy_to(target)
    torch.cuda.synchronize()
    assert torch.equal(target["w"], got["w"]) and torch.equal(target["b"], got["b"])
    with pytest.raises(L.EriError, match="No EMA weights found for parameter: nope"):
        ema.copy_to({"nope": torch.zeros(4, device="cuda")})
