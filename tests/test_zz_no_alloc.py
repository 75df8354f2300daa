"""``nrl_grpo_loss_fwd_bwd_static`` (the entry point that allocates nothing: its per-sequence partial sums
live in a fixed device array inside the library) against ``nrl_grpo_loss_fwd_bwd`` with a caller workspace,
through the C ABI, bit for bit.  Two calls in a row, the second on a smaller batch, so that what the first
call left in the shared array is shown not to leak into the second."""

import ctypes as C

import pytest
import torch

from rl_amd import _lib

pytestmark = pytest.mark.gpu


def _ptr(t):
    return C.c_void_p(0 if t is None else t.data_ptr())


def _inputs(batch, sm1, seed, dev):
    g = torch.Generator().manual_seed(seed)
    lp = -torch.rand(batch, sm1, generator=g) * 3.0
    t = {
        "lp": lp,
        "prev": lp + 0.05 * torch.randn(batch, sm1, generator=g),
        "ref": lp + 0.05 * torch.randn(batch, sm1, generator=g),
        "adv": torch.randn(batch, 1, generator=g).expand(batch, sm1).contiguous(),
        "token_mask": (torch.rand(batch, sm1, generator=g) < 0.7).float(),
        "sample_mask": (torch.rand(batch, generator=g) < 0.9).float(),
    }
    t["gen"] = t["prev"] + 0.01 * torch.randn(batch, sm1, generator=g)
    t = {k: v.to(dev) for k, v in t.items()}
    mask = t["token_mask"] * t["sample_mask"].unsqueeze(-1)
    t["global_valid"] = torch.stack([t["sample_mask"].sum(), mask.sum()]).float()
    return t


def _structs(t, batch, sm1, token_level):
    cfg = _lib.NrlGrpoCfg()
    cfg.token_level_loss = int(token_level)
    cfg.kl_type, cfg.has_kl, cfg.has_kl_input_clamp, cfg.has_kl_output_clamp = 3, 1, 1, 1
    cfg.ratio_clip_min, cfg.ratio_clip_max, cfg.kl_beta = 0.2, 0.28, 0.01
    cfg.kl_input_clamp, cfg.kl_output_clamp = 20.0, 10.0
    inp = _lib.NrlGrpoInputs()
    inp.batch, inp.sm1 = batch, sm1
    for name in ("lp", "prev", "gen", "ref", "adv", "token_mask"):
        setattr(inp, name, t[name].data_ptr())
        setattr(inp, name + "_stride", sm1)
    inp.lpu, inp.lpu_stride = 0, 0
    inp.sample_mask = t["sample_mask"].data_ptr()
    inp.correct_mask = 0
    inp.global_valid = t["global_valid"].data_ptr()
    return cfg, inp


def _outputs(batch, sm1, dev):
    return (torch.full((1,), float("nan"), device=dev), torch.full((batch, sm1), float("nan"), device=dev),
            torch.full((_lib.NRL_GRPO_N_METRICS,), float("nan"), device=dev))


def _run_pair(lib, batch, sm1, seed, token_level, dev):
    t = _inputs(batch, sm1, seed, dev)
    cfg, inp = _structs(t, batch, sm1, token_level)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    # every buffer exists before the call under test: that call must not need the allocator
    loss_w, dlp_w, met_w = _outputs(batch, sm1, dev)
    loss_s, dlp_s, met_s = _outputs(batch, sm1, dev)
    ws_bytes = lib.nrl_grpo_loss_workspace_bytes(batch)
    ws = torch.empty(ws_bytes // 8, dtype=torch.float64, device=dev)
    torch.cuda.synchronize()
    # free bytes of the device as the driver reports them: unlike torch's own counters this also sees a hipMalloc
    # made inside the library (the first call on a device, which resolves the array's address, came before)
    before = torch.cuda.mem_get_info()[0]
    code = lib.nrl_grpo_loss_fwd_bwd_static(C.byref(cfg), C.byref(inp), _ptr(loss_s), _ptr(dlp_s), None, _ptr(met_s), stream)
    _lib.check(code, "nrl_grpo_loss_fwd_bwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == before
    code = lib.nrl_grpo_loss_fwd_bwd(C.byref(cfg), C.byref(inp), _ptr(loss_w), _ptr(dlp_w), None, _ptr(met_w),
                                     _ptr(ws), ws_bytes, stream)
    _lib.check(code, "nrl_grpo_loss_fwd_bwd")
    torch.cuda.synchronize()
    assert torch.isfinite(loss_s).all() and loss_s.abs().item() > 0
    assert torch.equal(loss_s, loss_w)
    assert torch.equal(dlp_s, dlp_w)
    assert torch.equal(met_s, met_w)
    return loss_s.item()


def _warm_up(lib, dev):
    """The first call on a device resolves the address of the library's array (and loads its code object)."""
    t = _inputs(2, 3, 1, dev)
    cfg, inp = _structs(t, 2, 3, True)
    loss, dlp, met = _outputs(2, 3, dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.nrl_grpo_loss_fwd_bwd_static(C.byref(cfg), C.byref(inp), _ptr(loss), _ptr(dlp), None, _ptr(met), stream),
               "nrl_grpo_loss_fwd_bwd_static")
    torch.cuda.synchronize()


def test_static_scratch_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    with torch.cuda.device(dev):
        _warm_up(lib, dev)
        first = _run_pair(lib, 192, 511, seed=11, token_level=False, dev=dev)
        second = _run_pair(lib, 24, 200, seed=12, token_level=False, dev=dev)   # smaller: stale rows 24..191 stay behind
        third = _run_pair(lib, 7, 33, seed=13, token_level=True, dev=dev)
    assert len({first, second, third}) == 3


def test_static_scratch_calls_back_to_back_on_one_stream_without_a_host_wait():
    """Calls in stream order share the array safely: a large batch immediately followed by a smaller one, no
    synchronisation in between, each bit-equal to the workspace entry point on the same inputs."""
    lib = _lib.load()
    dev = torch.device("cuda:0")
    with torch.cuda.device(dev):
        _warm_up(lib, dev)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        cases = []
        for batch, sm1, seed in ((4096, 257, 21), (40, 129, 22), (1, 5, 23)):
            t = _inputs(batch, sm1, seed, dev)
            cfg, inp = _structs(t, batch, sm1, False)
            ws_bytes = lib.nrl_grpo_loss_workspace_bytes(batch)
            ws = torch.empty(ws_bytes // 8, dtype=torch.float64, device=dev)
            cases.append((t, cfg, inp, _outputs(batch, sm1, dev), _outputs(batch, sm1, dev), ws, ws_bytes))
        torch.cuda.synchronize()
        free = torch.cuda.mem_get_info()[0]
        for t, cfg, inp, (loss_s, dlp_s, met_s), _, _, _ in cases:          # nothing but launches in between
            _lib.check(lib.nrl_grpo_loss_fwd_bwd_static(C.byref(cfg), C.byref(inp), _ptr(loss_s), _ptr(dlp_s), None,
                                                        _ptr(met_s), stream), "nrl_grpo_loss_fwd_bwd_static")
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free
        for t, cfg, inp, (loss_s, dlp_s, met_s), (loss_w, dlp_w, met_w), ws, ws_bytes in cases:
            _lib.check(lib.nrl_grpo_loss_fwd_bwd(C.byref(cfg), C.byref(inp), _ptr(loss_w), _ptr(dlp_w), None, _ptr(met_w),
                                                 _ptr(ws), ws_bytes, stream), "nrl_grpo_loss_fwd_bwd")
            torch.cuda.synchronize()
            assert torch.isfinite(loss_s).all()
            assert torch.equal(loss_s, loss_w) and torch.equal(dlp_s, dlp_w) and torch.equal(met_s, met_w)


def test_static_scratch_entry_point_rejects_a_batch_beyond_its_array():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    batch, sm1 = _lib.NRL_GRPO_STATIC_MAX_BATCH + 1, 2
    with torch.cuda.device(dev):
        t = _inputs(batch, sm1, 5, dev)
        cfg, inp = _structs(t, batch, sm1, True)
        loss, dlp, met = _outputs(batch, sm1, dev)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        code = lib.nrl_grpo_loss_fwd_bwd_static(C.byref(cfg), C.byref(inp), _ptr(loss), _ptr(dlp), None, _ptr(met), stream)
        assert code == -4
        assert b"static scratch" in lib.nrl_last_error()
        with pytest.raises(ValueError, match="exceeds"):
            _lib.check(code, "nrl_grpo_loss_fwd_bwd_static")
        # the limit itself is accepted
        batch = _lib.NRL_GRPO_STATIC_MAX_BATCH
        t = _inputs(batch, sm1, 6, dev)
        cfg, inp = _structs(t, batch, sm1, True)
        loss, dlp, met = _outputs(batch, sm1, dev)
        code = lib.nrl_grpo_loss_fwd_bwd_static(C.byref(cfg), C.byref(inp), _ptr(loss), _ptr(dlp), None, _ptr(met), stream)
        _lib.check(code, "nrl_grpo_loss_fwd_bwd_static")
        torch.cuda.synchronize()
        assert torch.isfinite(loss).all()
