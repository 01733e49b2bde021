"""The host layer used from C++: tests/cpp/host_api_check.cc includes graph.h, graph_ops.h,
tensor_ops.h and hetero_graph.h the way the reference's C++ tests include its headers
(tests/test_colwise_slicing.cc:1-3), links libgs.so and checks the operators against closed
forms.  Here: that it links and loads without a GPU, and that every check holds on one."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "host_api_check")


def _binary():
    if not os.path.exists(BINARY):
        from graph_sampling_amd import build
        build.build_cpp_check()
    return BINARY


def test_cpp_caller_links_and_loads():
    import torch
    if torch.cuda.is_available():
        pytest.skip("covered by the GPU run of the same program")
    p = subprocess.run([_binary()], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=300)
    assert p.returncode == 2, p.stdout
    assert "no GPU" in p.stdout


@pytest.mark.gpu
def test_cpp_caller_passes_every_check(dev):
    p = subprocess.run([_binary()], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=300)
    print(p.stdout)
    assert p.returncode == 0, p.stdout
    assert p.stdout.strip().endswith("ALL OK"), p.stdout
