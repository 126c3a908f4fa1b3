"""Host-only checks around the layer-list worker class: the library profile that holds this class alone builds and carries every
entry point the host engine and the trace tool call; the oracle's own mechanisms agree with each other where two of them
describe the same thing."""
import ctypes as C
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import gelarax_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_layered_only_library_builds_and_declines_the_standard_network():
    from inferflow_amd import build
    path = build.build_layered_library()
    assert os.path.exists(path) and os.path.exists(build.LAYERED_CLI_PATH)
    # in a process of its own: another test may have loaded the full library with RTLD_GLOBAL, and its symbols would answer first
    code = ("import ctypes as C, sys\n"
            "L = C.CDLL(sys.argv[1])\n"
            "names = sys.argv[2].split(',')\n"
            "missing = [n for n in names if not hasattr(L, n)]\n"
            "L.ifa_last_error.restype = C.c_char_p\n"
            "out = C.c_void_p()\n"
            "rc = L.ifa_model_create(None, C.byref(out))\n"
            "print(missing, rc, L.ifa_last_error().decode())\n")
    names = ("ifa_model_create_layered", "ifa_model_set_tensor_host", "ifa_model_step_seqs", "ifa_model_logits_f32", "ifa_model_forward",
             "ifa_model_decode", "ifa_model_decode_batch", "ifa_model_kv_slots", "ifa_model_select_kv", "ifa_model_finalize", "ifa_model_destroy",
             "ifa_engine_create_from_dir", "ifa_engine_infer", "ifa_engine_commit", "ifa_engine_last_logits_f32", "ifa_linear_bf16w",
             "ifa_attention_window_f32", "ifa_state_scan_f32", "ifa_shortconv_silu_f32", "ifa_dyt_f32", "ifa_add_dyt_f32", "ifa_embed_pair_scaled_f32",
             "ifa_qkv_rope_store_f32", "ifa_rotate_heads_f32", "ifa_attention_kv_sinks_f32", "ifa_chan_delta_gates_f32", "ifa_state_scan_chan_f32",
             "ifa_moe_dyt_route_rows_f32", "ifa_moe_experts_glu_f32")
    r = subprocess.run([sys.executable, "-c", code, path, ",".join(names)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.startswith("[] -4 ") and "standard network" in r.stdout, r.stdout
    assert os.access(os.path.join(ROOT, "bin", "trace_run"), os.X_OK)


def test_oracle_bucket_map_and_visibility():
    assert [orc.distance_bucket(n, 8, 32) for n in (0, 1, 3, 4, 5, 31, 32, 500)] == [0, 1, 3, 4, 4, 7, 7, 7]
    rows = [orc.distance_bucket(n, 24, 100) for n in range(300)]
    assert rows[:12] == list(range(12)) and all(b >= a for a, b in zip(rows, rows[1:])) and rows[100] == 23 and rows[99] == 23 and max(rows) == 23
    v = orc.visible(12, 4, 2).numpy()
    assert v[11].tolist() == [True, True] + [False] * 6 + [True] * 4 and v[3].tolist() == [True] * 4 + [False] * 8


def test_oracle_recurrences_against_their_closed_forms():
    rng = np.random.default_rng(0)
    T, dk, dv = 9, 5, 3
    q, k, v = (orc.t64(rng.standard_normal((T, n))) for n in (dk, dk, dv))
    d = 0.8
    got = orc.decayed_linear_attention(q, k, v, 1, dk, dv, orc.t64([d]))
    want = torch.stack([sum(d ** (t - j) * (q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(T)])
    assert torch.allclose(got, want, atol=1e-12)
    # delta rule with beta = 1, g = 1 and orthonormal keys stores each value exactly: reading with k_j returns v_j
    kk = torch.eye(dk, dtype=orc.F64)[:4]
    vv = orc.t64(rng.standard_normal((4, dv)))
    o = orc.gated_delta_rule(kk, kk, vv, torch.ones(4, 1, dtype=orc.F64), torch.ones(4, 1, dtype=orc.F64), 1, 1, dk, dv)
    assert torch.allclose(o, vv, atol=1e-12)
    # a one-tap convolution is a per-channel scale
    x, w = orc.t64(rng.standard_normal((6, 4))), orc.t64(rng.standard_normal((4, 1)))
    assert torch.allclose(orc.short_conv(x, w), x * w[:, 0])
