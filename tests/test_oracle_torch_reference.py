"""The PyTorch restatement of the upstream tests' reference (oracle/torch_reference.py, what bench.py
times on the host cores) against the C oracle, and its two forms against each other."""
import pytest
import torch

from flash_attention_factory_amd import workloads as W
from oracle import torch_reference as T
from _torch_ref import call_oracle, sdpa_reference

CASES = [
    ("config0", lambda: W.make_config(0)),
    ("config1_small_token_major", lambda: W.make_config(1, num_seqs=3, pool_blocks=400, layout=W.TOKEN_MAJOR)),
    ("config3_small", lambda: W.make_config(3, num_seqs=3, pool_blocks=400)),
    ("config4_small", lambda: W.make_config(4, num_seqs=4, pool_blocks=2048, lens=[64, 700, 0, 1300])),
    ("grid_sinks", lambda: W.make_test_shaped(batch_size=2, nheads=10, nheads_k=2, d=64, seqlen_k=339, varlen=True,
                                              has_sinks=True)),
    ("grid_fp8_e4m3", lambda: W.make_test_shaped(batch_size=2, nheads=8, nheads_k=2, d=128, seqlen_k=200, varlen=True,
                                                 has_sinks=True, fp8=True, fp8_dtype=torch.float8_e4m3fn)),
]


@pytest.mark.parametrize("name,make", CASES, ids=[c[0] for c in CASES])
def test_torch_reference_equals_the_c_oracle(oracle, name, make):
    w = make()
    ref16, ref32 = call_oracle(oracle.attention_ref, w, want_f32=True)
    per_seq = T.run_workload(w)
    live = w.context_lens > 0
    assert (per_seq[~live] == 0).all()
    ulp = 2.0 ** (-8 if w.query.dtype == torch.bfloat16 else -11)
    scale = ref32.abs().max()
    # both round an fp32 result once; fp32 summation orders differ, so allow one unit in the last place
    assert ((per_seq.float() - ref16.float()).abs().max() <= 1.01 * ulp * scale)
    if live.all():
        padded = T.run_workload(w, padded=True)
        assert ((padded.float() - ref16.float()).abs().max() <= 1.01 * ulp * scale)
        if w.query.dtype == torch.float16 or not w.is_fp8:
            torch.testing.assert_close(padded.float(), sdpa_reference(w), atol=2 * ulp * float(scale), rtol=0)


def test_padded_form_size():
    w = W.make_config(0)
    S, H, D = w.query.shape
    assert T.padded_bytes(w) == 2 * S * int(w.context_lens.max()) * H * D * 4
