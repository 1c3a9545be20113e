"""The entry point that allocates nothing (plk_mok_forward_static), called through the C ABI: its outputs equal
plk_mok_forward's byte for byte on two calls in a row, the second with a smaller input (the library's fixed device
area still holds the first call's params images and workspace then).  The first problem's rows of hidden_q are whole
cache lines (one launch, readiness counters in the fixed area), the second's are not (two launches)."""
import json

import pytest
import torch

pytestmark = pytest.mark.gpu


def _device_problem(sess, inp, H, I, pitch_i=None):
    from pipelink_amd.host.mok import scale_pitch, weight_codes_to_k64_tiled, weight_scales_to_slot_major

    dev = torch.device("cuda:0")
    d = {k: v.to(dev) for k, v in inp.__dict__.items()}
    d["w_gate_sc"] = weight_scales_to_slot_major(d["w_gate_sc"], H)
    d["w_up_sc"] = weight_scales_to_slot_major(d["w_up_sc"], H)
    d["w_down_sc"] = weight_scales_to_slot_major(d["w_down_sc"], I)
    d["w_gate_q"] = weight_codes_to_k64_tiled(d["w_gate_q"], H)
    d["w_up_q"] = weight_codes_to_k64_tiled(d["w_up_q"], H)
    d["w_down_q"] = weight_codes_to_k64_tiled(d["w_down_q"], I)
    rows = int(inp.tokens_per_expert.sum())
    out = dict(hidden_q=torch.empty((rows, pitch_i or I), dtype=torch.uint8, device=dev),
               hidden_sc=torch.empty((rows, scale_pitch(I)), dtype=torch.uint8, device=dev),
               y=torch.empty((rows, H), dtype=torch.bfloat16, device=dev))
    return sess.problem(**out, **d), out, d  # d keeps the input tensors alive


def _poison(out):
    out["hidden_q"].fill_(0xFF)
    out["hidden_sc"].fill_(0xFF)
    out["y"].fill_(float("nan"))


def _snapshot(out):
    torch.cuda.synchronize()
    return [out["hidden_q"].cpu(), out["hidden_sc"].cpu(), out["y"].view(torch.int16).cpu()]


def test_static_entry_point_matches_forward_on_two_calls_in_a_row():
    from pipelink_amd.host import mok_inputs
    from pipelink_amd.host.mok import MoKSession
    from pipelink_amd.stages.mok import build as mok_build

    paths = mok_build.images()
    link = json.loads(paths["link_json"].read_text())
    shapes = [(700, 448, 704, 6, 2, 21, 768), (96, 256, 320, 8, 2, 22, None)]  # T, H, I, E, top_k, seed, pitch of hidden_q
    with MoKSession(paths["linked"].read_bytes(), link) as sess:
        cases = []
        for T, H, I, E, k, seed, pitch in shapes:
            inp = mok_inputs.generate(T, H, I, E, k, seed=seed)
            cases.append(_device_problem(sess, inp, H, I, pitch))
        expected = []
        for prob, out, _ in cases:
            _poison(out)
            sess.forward(prob)
            expected.append(_snapshot(out))
        for prob, out, _ in cases:
            _poison(out)
        torch.cuda.synchronize()
        for prob, out, _ in cases:  # back to back on one stream, no host wait between them
            sess.forward_static(prob)
        assert sess.status() == 0
        for (prob, out, _), want in zip(cases, expected):
            got = _snapshot(out)
            for g, w in zip(got, want):
                assert torch.equal(g, w)
            assert not torch.isnan(out["y"].float()).any()


def test_static_entry_point_allocates_nothing_and_can_be_captured():
    """What the entry point is for: the device's free memory is the same after the calls as before them (no hipMalloc /
    hipFree, by the library or by torch), and two calls in a row are captured into a HIP graph on a fresh stream -- a
    new problem each, where plk_mok_forward would have to upload an image and says PLK_E_CONTRACT -- and every replay
    writes the bytes of the eager forward."""
    from pipelink_amd.host import mok_inputs
    from pipelink_amd.host.backend import HipBackend, PlkError
    from pipelink_amd.host.mok import MoKSession
    from pipelink_amd.stages.mok import build as mok_build

    paths = mok_build.images()
    link = json.loads(paths["link_json"].read_text())
    shapes = [(520, 320, 384, 4, 2, 31, 384), (96, 256, 320, 8, 2, 32, None)]
    with MoKSession(paths["linked"].read_bytes(), link) as sess, MoKSession(paths["linked"].read_bytes(), link) as fresh:
        cases = [_device_problem(sess, mok_inputs.generate(T, H, I, E, k, seed=seed), H, I, pitch) for T, H, I, E, k, seed, pitch in shapes]
        expected = []
        for prob, out, _ in cases:
            _poison(out)
            sess.forward(prob)
            expected.append(_snapshot(out))
        for prob, out, _ in cases:
            _poison(out)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for prob, out, _ in cases:
            sess.forward_static(prob)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        for (prob, out, _), want in zip(cases, expected):
            assert all(torch.equal(g, w) for g, w in zip(_snapshot(out), want))

        be = HipBackend(0, 0)
        stream = be.stream_create()
        # a session that has never seen these problems: plk_mok_forward would have to upload their params images
        with pytest.raises(PlkError):
            be.capture(stream, lambda: fresh.forward(cases[0][0], stream=stream))

        def body():
            for prob, out, _ in cases:
                fresh.forward_static(prob, stream=stream)

        graph = be.capture(stream, body)
        try:
            for replay in range(3):
                for prob, out, _ in cases:
                    _poison(out)
                torch.cuda.synchronize()   # the program's own eager work and synchronisation between the replays
                graph.launch(stream)
                be.synchronize(stream)
                for (prob, out, _), want in zip(cases, expected):
                    assert all(torch.equal(g, w) for g, w in zip(_snapshot(out), want)), f"replay {replay}"
            assert fresh.status() == 0
        finally:
            graph.close()
            be.close()


def test_static_entry_point_rejects_sizes_beyond_its_area():
    from ctypes import sizeof

    from pipelink_amd.host import mok_inputs
    from pipelink_amd.host.backend import MokLinkInfo, PlkError
    from pipelink_amd.host.mok import MoKSession, link_info_from_json
    from pipelink_amd.stages.mok import build as mok_build

    paths = mok_build.images()
    info = link_info_from_json(json.loads(paths["link_json"].read_text()))
    big = MokLinkInfo(struct_bytes=sizeof(MokLinkInfo), params_bytes=2048, framework_offset=info.framework_offset,
                      gemm_offset=info.gemm_offset, act_offset=info.act_offset, threads=info.threads,
                      dyn_lds_bytes=info.dyn_lds_bytes, workgroups_per_cu=info.workgroups_per_cu)
    with MoKSession(paths["linked"].read_bytes(), big) as sess:
        inp = mok_inputs.generate(64, 64, 64, 2, 1, seed=0)
        prob, out, _ = _device_problem(sess, inp, 64, 64)
        with pytest.raises(PlkError) as err:
            sess.forward_static(prob)
        assert err.value.status == 2  # PLK_E_CAPACITY
