"""Host-side logic that needs no GPU: synthetic input generators, the drop-in import path, and the loud failure
of the classifier module when no GPU device is configured."""
import types

import numpy as np
import pytest

from elmo_amd import synth


def test_make_x_rows_are_unit_norm_bf16():
    x = synth.make_x(32, 768, 0)
    assert x.shape == (32, 768) and x.dtype == np.float32
    assert np.all((x.view(np.uint32) & 0xFFFF) == 0)                 # bf16 values
    assert np.allclose(np.linalg.norm(x, axis=1), 1.0, atol=5e-3)
    assert np.array_equal(x, synth.make_x(32, 768, 0)) and not np.array_equal(x, synth.make_x(32, 768, 1))


def test_make_labels_format_and_distribution():
    lab = synth.make_labels(128, 670091, 5.4, 1.0, 1)
    assert lab.dtype == np.int32 and lab.ndim == 2 and lab.shape[1] == 2
    assert lab[:, 0].min() >= 0 and lab[:, 0].max() < 128 and lab[:, 1].min() >= 0 and lab[:, 1].max() < 670091
    assert np.all(np.diff(lab[:, 0]) >= 0)                            # row-major, as the reference's collate emits
    assert len(np.unique(lab, axis=0)) == len(lab)                    # de-duplicated within a row
    assert 3.5 < len(lab) / 128 < 7.5                                 # Poisson(5.4) minus collisions
    head = np.mean(lab[:, 1] < 1000)
    assert 0.3 < head < 0.7                                           # Zipf(1.0): about half of the mass in the first 1000 ranks
    empty = synth.make_labels(4, 100, 0.0, 1.0, 0)
    assert empty.shape == (0, 2)


def test_configs_cover_the_five_benchmark_shapes():
    c = synth.CONFIGS
    assert c["cfg2_fp8_670k"].num_labels == 670091 and c["cfg2_fp8_670k"].batch == 128 and c["cfg2_fp8_670k"].num_chunks == 11
    assert c["cfg1_bf16_131k"].num_chunks == 8 and c["cfg4_fp8_3m"].num_chunks == 22 and c["cfg5_fp8_8m6"].num_chunks == 33


def test_reference_import_paths_resolve():
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    from elmo_amd.xmc_classifiers import Fp8XMCBCEChunkedLayer as Same
    assert Fp8XMCBCEChunkedLayer is Same
    for name in ("xfc_forward", "xfc_forward_backward", "filter_non_local_inds", "_compute_loss"):
        assert callable(getattr(Fp8XMCBCEChunkedLayer, name))


def make_cfg(device, num_labels=1000, num_chunks=2, simulated=False, **xmc_extra):
    ns = types.SimpleNamespace
    return ns(environment=ns(device=device), data=ns(num_labels=num_labels, batch_size=32),
              model=ns(xmc=ns(num_chunks=num_chunks, input_features=768, dtype="float8")),
              training=ns(xmc=ns(simulated_fp8=simulated, momentum=0, wd=0, **xmc_extra),
                          precision=ns(mode="custom", purelp_dtype="bfloat16")))


def test_module_refuses_to_run_without_a_gpu():
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    with pytest.raises(AssertionError):
        Fp8XMCBCEChunkedLayer(make_cfg("cpu"))


def test_bench_rejects_more_than_one_gpu():
    import subprocess, sys, os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr
