"""The sweep and block scripts under triton-kernels_amd/benchmarks run and agree with PyTorch at the
reference scripts' ragged shapes (scripts/single_triton.py:13-14: batch 3 x 4336 tokens;
scripts/double_triton.py:12-15: 4080 img + 256 txt tokens, neither a multiple of a tile)."""
import pytest
import torch

from benchmarks import blocks, sweep
from util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", list(sweep.OPS))
def test_sweep_rows(name, tmp_path):
    timer = sweep.Timer(torch.device(DEV), reps=2, warmup=1, flush_mb=0)
    for mode in sweep.OPS[name][2]:
        rows = sweep.run_op(name, mode, [192], 2, timer, torch.device(DEV), out_dir=str(tmp_path), echo=lambda s: None)
        assert rows[0]["seq_len"] == 192 and rows[0]["hip_ms"] > 0 and rows[0]["torch_ms"] > 0
        assert (tmp_path / mode / (sweep.OPS[name][3] + ".csv")).read_text().startswith("seq_len,hip_ms,hip_gbps")


@pytest.mark.parametrize("kind", ["single", "double"])
def test_block_scripts_ragged_shapes(kind):
    plain, hip = blocks.build_pair(kind, 3072, 24, 4.0, DEV, seed=7)
    torch.manual_seed(11)
    inputs = blocks.make_inputs(kind, 3, 4336, 4080, 256, 3072, 24, DEV)
    worst = blocks.compare(plain, hip, inputs, atol=0.1)
    assert worst < 0.1
    assert blocks.time_block(hip, inputs, warmup=1, runs=2) > 0
