"""One whole UNet step of the path (BASELINE config 5) checked end to end against the oracle.

The C++ step runner enqueues the 133 launches of a step in the reference's call order
(M/UNetModel.cpp:1078-1929: timestep embedding, the SiLU of the time-embedding MLP, per ResBlock
GroupNorm+SiLU / SiLU(emb) / GroupNorm+SiLU in place (M/nn/ResBlock.cpp:125-232), per transformer
block three LayerNorms and the GEGLU epilogue (M/nn/BasicTransformerBlock.cpp:116-164), and the
final GroupNorm+SiLU (M/UNetModel.cpp:1796-1810)), batch 2, fp16 storage.  Every one of the 133
outputs is read back and compared with the oracle applied to the very input the launch saw:
after an eager run, after the 1st replay of the captured graph and after the 25th, the sampler's
integer timesteps (M/DDIMSampler.cpp:60-64,78-82) walked from the back.
"""
import ctypes

import numpy as np
import pytest

from tolerances import assert_close_f16

pytestmark = pytest.mark.gpu

KINDS = {0: "gn_silu", 1: "layernorm", 2: "geglu", 3: "silu"}


def _download(nn, st, i, which):
    n = ctypes.c_size_t(0)
    assert nn.msdnn_step_download(st, i, which, None, 0, ctypes.byref(n)) == 0
    out = np.empty(n.value, dtype=np.float32)
    assert nn.msdnn_step_download(st, i, which, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), n.value,
                                  None) == 0
    return out


def _all_outputs(nn, st, n_ops):
    return [_download(nn, st, i, 1) for i in range(n_ops)], _download(nn, st, 0, 2)


def test_config5_step_outputs_match_oracle_eager_and_after_graph_replays(msd, orc, cuda):
    import torch
    nn = msd.load_nn_library()
    stream = torch.cuda.Stream()
    sp = ctypes.c_void_p(stream.cuda_stream)
    batch = 2
    st = nn.msdnn_step_create(sp, batch, msd.DTYPE_F16, 1)
    assert st, msd.nn_last_error()
    try:
        n_ops = nn.msdnn_step_num_ops(st)
        assert n_ops + 1 == nn.msdnn_step_launches(st) == 133
        assert nn.msdnn_step_bytes(st) == 1099694080

        # what each launch works on, its pristine input and its affine, before anything has run
        infos, inputs, affines = [], [], []
        counts = {k: 0 for k in KINDS.values()}
        for i in range(n_ops):
            kind, in_place = ctypes.c_int(0), ctypes.c_int(0)
            dims = (ctypes.c_size_t * 2)()
            assert nn.msdnn_step_op_info(st, i, ctypes.byref(kind), dims, ctypes.byref(in_place)) == 0
            infos.append((KINDS[kind.value], int(dims[0]), int(dims[1]), bool(in_place.value)))
            counts[KINDS[kind.value]] += 1
            inputs.append(_download(nn, st, i, 0))
            if kind.value in (0, 1):
                c = int(dims[0]) if kind.value == 0 else int(dims[1])
                g, b = np.empty(c, np.float32), np.empty(c, np.float32)
                fp = ctypes.POINTER(ctypes.c_float)
                assert nn.msdnn_step_affine(st, i, g.ctypes.data_as(fp), b.ctypes.data_as(fp), c) == c
                affines.append((g, b))
            else:
                affines.append(None)
        assert counts == {"gn_silu": 45, "layernorm": 48, "geglu": 16, "silu": 23}

        # the oracle on the same inputs (fp32 arithmetic on the stored fp16 values), unrounded
        refs = []
        for (kind, d0, d1, _), x, ab in zip(infos, inputs, affines):
            if kind == "gn_silu":
                refs.append(orc.groupnorm(x.reshape(batch, d0, d1), ab[0], ab[1], 32, 1e-5, silu=True).reshape(-1))
            elif kind == "layernorm":
                refs.append(orc.layernorm(x.reshape(d0, d1), ab[0], ab[1], 1e-5).reshape(-1))
            elif kind == "geglu":
                refs.append(orc.geglu(x.reshape(d0, 2 * d1)).reshape(-1))
            else:
                refs.append(orc.silu(x))

        sched = msd.ddim_timesteps(25)[::-1]  # 961, 921, ..., 1
        assert sched == orc.ddim_timesteps(25)[::-1] and len(sched) == 25

        def check_embedding(emb, t):
            ref = np.stack([orc.timestep_embedding(t)] * batch).reshape(-1)
            assert_close_f16(emb, ref, "cfg5 step: timestep embedding")

        # ---- eager
        ts = (ctypes.c_long * batch)(*([sched[0]] * batch))
        assert nn.msdnn_step_run(st, 1, 0, ts, batch) == 0, msd.nn_last_error()
        assert msd.load_library().msd_status(sp) == 0
        eager, emb = _all_outputs(nn, st, n_ops)
        check_embedding(emb, sched[0])
        for i, ((kind, d0, d1, _), got, ref) in enumerate(zip(infos, eager, refs)):
            assert_close_f16(got, ref, "cfg5 step: %s %dx%d" % (kind, d0, d1))

        # ---- 25 replays of the captured graph, one timestep of the schedule each; inputs that
        # in-place layers overwrote are put back (eager copies) between replays
        for k, t in enumerate(sched):
            assert nn.msdnn_step_restore(st) == 0, msd.nn_last_error()
            ts = (ctypes.c_long * batch)(*([t] * batch))
            assert nn.msdnn_step_run(st, 1, 1, ts, batch) == 0, msd.nn_last_error()
            if k in (0, len(sched) - 1):
                assert msd.load_library().msd_status(sp) == 0
                outs, emb = _all_outputs(nn, st, n_ops)
                check_embedding(emb, t)
                # the kernels are deterministic, so a replay must reproduce the eager outputs
                # (already checked against the oracle above) bit for bit
                for i, (got, want) in enumerate(zip(outs, eager)):
                    assert np.array_equal(got, want), "replay %d: output of launch %d (%s) differs from eager" % (
                        k + 1, i + 1, infos[i][0])
    finally:
        nn.msdnn_step_destroy(st)
