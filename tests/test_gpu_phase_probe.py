"""The timestamping instantiation of the decode GEMV (oxq_set_gemv_phase_probe, include/oxq_tuning.h): same
results as the plain launch, one record per wave, timestamps in order."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q4_K, Q6_K, Q8_0 = 12, 14, 8


@pytest.mark.parametrize("qtype,n_rows,n_cols", [(Q8_0, 1024, 4096), (Q4_K, 2048, 4096), (Q6_K, 512, 14336)])
def test_probe_same_bits_and_ordered_stamps(hip, qtype, n_rows, n_cols):
    import torch
    from oxillama_amd import capi, synth
    lib = capi.load()
    dev = torch.device("cuda:0")
    w = torch.from_numpy(synth.weights(qtype, 11, n_rows, n_cols)).to(dev)
    aq = torch.empty(n_cols // 32 * 34, dtype=torch.uint8, device=dev)
    hip.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(3, n_cols)).to(dev), aq)
    k = hip.HipKernel(qtype)
    plain = torch.zeros(n_rows, device=dev)
    k.matvec_q8_fused_dev(w, aq, plain, n_rows, n_cols, accumulate=False)
    cap = 1 << 20
    buf = torch.zeros(cap // 8, dtype=torch.int64, device=dev)
    probed = torch.zeros(n_rows, device=dev)
    assert lib.oxq_set_gemv_phase_probe(buf.data_ptr(), cap) == capi.OK
    try:
        k.matvec_q8_fused_dev(w, aq, probed, n_rows, n_cols, accumulate=False)
        torch.cuda.synchronize()
    finally:
        lib.oxq_set_gemv_phase_probe(None, 0)
    assert np.array_equal(plain.cpu().numpy().view(np.uint32), probed.cpu().numpy().view(np.uint32))
    rec = buf.cpu().numpy().reshape(-1, 4)
    rec = rec[rec[:, 0] != 0]
    assert len(rec) > 0 and len(rec) % 4 == 0  # whole work groups of four waves
    assert (rec[:, 0] <= rec[:, 1]).all() and (rec[:, 1] <= rec[:, 2]).all()
    # a buffer too small for the launch: the plain kernel runs, nothing is written
    buf.zero_()
    assert lib.oxq_set_gemv_phase_probe(buf.data_ptr(), 64) == capi.OK
    try:
        k.matvec_q8_fused_dev(w, aq, probed, n_rows, n_cols, accumulate=False)
        torch.cuda.synchronize()
    finally:
        lib.oxq_set_gemv_phase_probe(None, 0)
    assert int(buf.abs().sum().item()) == 0
