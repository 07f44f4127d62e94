"""The two host bindings of the C ABI - the compiled `deep_ep._C` extension (default) and the Python runtime over
ctypes - give the same results.  The rest of the GPU suite runs on whichever binding DEEP_EP_HIP_BINDING selects (the
compiled one by default); here the other one is started in a child process and checked against the oracle."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import os, sys
for sub in ("deepep-ascend_amd", "oracle", "tests"):
    sys.path.insert(0, os.path.join(%(root)r, sub))
import torch
import deep_ep
import routing_cases as rc
import routing_oracle as oracle
from test_gpu_parity import assert_equal
assert deep_ep._binding.name == %(binding)r, deep_ep._binding.name
case = rc.small("binding", 777, 1024, 32, 4, 6, seed=5, masked_ratio=0.1)
buf = deep_ep.ElasticBuffer(deep_ep.LogicalGroup(1, case.R), num_max_tokens_per_rank=case.M, hidden=case.H, num_topk=case.K)
x, idx, w = case.x.cuda(), case.topk_idx.cuda(), case.topk_weights.cuda()
for do_cpu_sync in (True, False):
    for do_expand in (False, True):
        ref = oracle.dispatch(oracle.per_token_cast_to_fp8(case.x), case.topk_idx, case.topk_weights, case.E, case.R, 1, case.M,
                              do_expand=do_expand, expert_alignment=4)
        (rx, rsf), ridx, rw, handle, ev = buf.dispatch(x, idx, w, num_experts=case.E, cast_to_fp8=True, do_expand=do_expand,
                                                       expert_alignment=4, do_cpu_sync=do_cpu_sync, do_zero_padding=do_expand,
                                                       async_with_compute_stream=True)
        ev.current_stream_wait()
        n = ref.num_expanded_tokens if do_expand else ref.num_recv_tokens
        assert_equal(rx[:n], ref.recv_x, "recv_x")
        assert_equal(rsf[:n], ref.recv_sf, "recv_sf")
        assert_equal(handle.dst_buffer_slot_idx, ref.dst_buffer_slot_idx, "dst_buffer_slot_idx")
        assert_equal(handle.recv_src_metadata[:ref.num_recv_tokens], ref.recv_src_metadata, "recv_src_metadata")
        y = oracle.per_token_cast_back(ref.recv_x, ref.recv_sf)
        ypad = torch.zeros((rx.shape[0], case.H), dtype=torch.bfloat16)
        ypad[:n] = y
        out, out_w, _ = buf.combine(ypad.cuda(), handle, topk_weights=rw)
        ref_out, ref_w = oracle.combine(y, case.topk_idx, ref.recv_src_metadata, ref.dst_buffer_slot_idx,
                                        ref.psum_num_recv_tokens_per_scaleup_rank, case.E, case.R, 1, case.M,
                                        topk_weights=ref.recv_topk_weights, do_expand=do_expand)
        assert_equal(out + 0.0, ref_out + 0.0, "combined_x")
        assert_equal(out_w, ref_w, "combined_topk_weights")
buf.check_device_status()
print("binding ok")
"""


@pytest.mark.parametrize("binding", ["ctypes", "pybind"])
def test_binding_in_a_child_process(binding):
    env = dict(os.environ, DEEP_EP_HIP_BINDING=binding)
    res = subprocess.run([sys.executable, "-c", CHILD % {"root": ROOT, "binding": binding}], env=env, capture_output=True,
                         text=True, timeout=300)
    assert res.returncode == 0 and "binding ok" in res.stdout, res.stdout[-2000:] + res.stderr[-4000:]
