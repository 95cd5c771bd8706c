"""GPU side of the retrain pass (nncp_retrain_block, dropout): the same host C
code as on the CPU checker, linked against libnc_hip.so.  Collected after the
other GPU tests (file name), so a failure here hides nothing else."""
import numpy as np
import pytest

import modelutil as M

pytestmark = [pytest.mark.gpu,
              pytest.mark.skip(reason="written without GPU access: to be enabled after its first run on an MI355X")]


@pytest.fixture(scope="module")
def hosts():
    return M.hip_host(), M.ref_host()


@pytest.mark.parametrize("fused", [0, 1])
def test_retrain_round_trip_on_gpu_and_size_against_checker(hosts, fused):
    pkg = M.load_pkg()
    cfg = dict(M.TINY, fused=fused, sgd_opt=M.rmsprop(), dropout_prob=0.1, dropout_att_prob=0.05,
               retrain_period=1)
    B, T = cfg["batch_size"], cfg["seg_len"]
    block = B * T * 3 + 5
    cfg["retrain_len"] = 2 * block
    syms = M.markov1(3 * block - 7, 40, seed=21)

    def model(host, dev):
        return pkg.host.Model(host, pkg.host.make_config(**dict(cfg, use_device=dev, nb_threads=4)))
    enc = model(hosts[0], 1)
    data, st, rst = enc.compress_blocks(syms, block, 1)
    w_enc = enc.params()
    enc.close()
    dec = model(hosts[0], 1)
    out, _, _ = dec.decompress_blocks(data, len(syms), block, 1)
    w_dec = dec.params()
    dec.close()
    assert np.array_equal(out, syms)
    for k in w_enc:
        assert np.array_equal(w_enc[k], w_dec[k]), k
    # the dropout masks come from the same host-side stream in both libraries, so the
    # checker follows the same trajectory up to fp32 reordering: size within 0.5 %
    ref = model(hosts[1], 0)
    data_ref, _, rst_ref = ref.compress_blocks(syms, block, 1)
    w_ref = ref.params()
    ref.close()
    assert rst.n_steps == rst_ref.n_steps > 0
    assert abs(len(data) - len(data_ref)) <= max(2, 0.005 * len(data_ref))
    for k in w_ref:
        assert M.tensors_close(w_enc[k], w_ref[k], 1e-5), (k, M.rel_l2(w_enc[k], w_ref[k]))
