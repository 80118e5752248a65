"""The C++ host mirror (weed_amd/host): its own test binary is built beforehand (tests/host/Makefile, run by
__graft_entry__.build()) and driven from here.  Host-logic cases run anywhere; the device cases need a GPU."""
import ctypes
import os
import subprocess

import pytest

from weed_amd import build as wb

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "host", "_build", "test_host_mirror")


def _run(args):
    if not os.path.exists(BINARY):
        pytest.fail("%s is missing: run __graft_entry__.build() (or make -C tests/host) first" % BINARY)
    proc = subprocess.run([BINARY] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-4000:]
    return proc.stdout


def test_host_library_loads_and_exports_the_mirror():
    path = wb.host_library_path()
    assert os.path.exists(path), "build the host mirror first (__graft_entry__.build())"
    ctypes.CDLL(wb.library_path(), mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(path)
    # a few mangled names of the mirrored interface: Weed::matmul, Weed::softmax, MultiHeadAttention::forward
    out = subprocess.run(["nm", "-DC", path], stdout=subprocess.PIPE, text=True, check=True).stdout
    for name in ("Weed::matmul(Weed::Tensor const&, Weed::Tensor const&, Weed::Tensor&)",
                 "Weed::softmax(unsigned int const&, Weed::Tensor const&, Weed::Tensor&)",
                 "Weed::reduce(unsigned int const&, Weed::Tensor const&, Weed::Tensor&)",
                 "Weed::MultiHeadAttention::forward(", "Weed::MultiHeadAttention::reset_cache()",
                 "Weed::QuantizedKVCache::write_row(unsigned int, float const*)",
                 "Weed::QuantizedKVCache::read_row(unsigned int, float*) const",
                 "Weed::Linear::forward(", "Weed::RMSNorm::forward(", "Weed::LayerNorm::forward(", "Weed::SwiGLU::forward(",
                 "Weed::QwenDecoderLayer::forward(", "Weed::TransformerEncoderLayer::forward(",
                 "Weed::MultiHeadAttention::set_tables(", "Weed::place_side_by_side(", "Weed::forward_side_by_side(",
                 "Weed::QwenDecoderLayer::fuse_projections()"):
        assert name in out, name
    assert lib is not None


def test_host_logic_without_a_device():
    out = _run(["--no-gpu"])
    assert "0 failed" in out


@pytest.mark.gpu
def test_host_mirror_on_device():
    out = _run([])
    assert "0 failed" in out and "test_attention_lloydmax" in out and "test_qwen_decoder_layer_prefill_then_decode" in out
    assert "test_projections_side_by_side" in out
