"""The unit state files: names, sizes and raw contents follow the reference's swap-file layout
(flextrain/memory/__init__.py:30-49, flextrain/memory/nvme_swapper.py:24-40,181-182,
flextrain/memory/coordinator/optimizer.py:219-235), worked out by hand here."""
import os

import numpy as np
import pytest
import torch

from flextrain_amd.state_files import (
    BACKWARD_SHARE, FORWARD_SHARE, FlexTrainDataID, FlexTrainDataType, opts_file_layout, opts_file_name,
    read_unit_opts, write_unit_opts,
)


def test_names():
    assert str(FlexTrainDataID(FlexTrainDataType.OPTS, 3)) == "rank0_OPTS_layer3.swp"
    assert str(FlexTrainDataID(FlexTrainDataType.PARA, 0, rank=5)) == "rank5_PARA_layer0.swp"
    # several layers per unit: the name carries the inclusive layer range
    assert str(FlexTrainDataID(FlexTrainDataType.OPTS, 3, checkpoint_interval=2)) == "rank0_OPTS_layer6-7.swp"
    assert str(FlexTrainDataID(FlexTrainDataType.CKPT, 0, rank=1, checkpoint_interval=4)) == "rank1_CKPT_layer0-3.swp"
    assert opts_file_name(7, FORWARD_SHARE) == "rank0_OPTS_layer7.swp.0"
    assert opts_file_name(7, BACKWARD_SHARE, rank=2) == "rank2_OPTS_layer7.swp.1"
    assert [t.value for t in FlexTrainDataType] == [0, 1, 2, 3]


def test_layout_sizes():
    # 1000 fp32 elements x 3 arrays = 12,000 bytes; the backward share is padded to 3 pages
    assert opts_file_layout(1000, FORWARD_SHARE) == (3000, 0, 12000)
    assert opts_file_layout(1000, BACKWARD_SHARE) == (3000, 72, 12288)
    # already page-aligned: 1024 x 3 x 4 = 12,288
    assert opts_file_layout(1024, BACKWARD_SHARE) == (3072, 0, 12288)
    # one element still occupies a page
    assert opts_file_layout(1, BACKWARD_SHARE) == (3, 1021, 4096)
    # SGD-with-momentum-like optimizer: one state per element; bf16 master: 2-byte items
    assert opts_file_layout(1000, BACKWARD_SHARE, states_per_element=1, itemsize=2) == (2000, 48, 4096)


@pytest.mark.parametrize("share", [FORWARD_SHARE, BACKWARD_SHARE])
@pytest.mark.parametrize("n", [1, 1000, 1024, 70_001])
def test_raw_contents_and_round_trip(tmp_path, share, n):
    rng = np.random.default_rng(n)
    blocks = [torch.from_numpy(rng.standard_normal(n).astype(np.float32)) for _ in range(3)]
    path = write_unit_opts(str(tmp_path), 4, blocks, share=share, rank=1)
    assert os.path.basename(path) == f"rank1_OPTS_layer4.swp.{share}"
    raw = np.fromfile(path, dtype="<f4")
    payload, padding, nbytes = opts_file_layout(n, share)
    assert os.path.getsize(path) == nbytes and raw.size == payload + padding
    assert np.array_equal(raw[:payload].view(np.uint32), np.concatenate([b.numpy() for b in blocks]).view(np.uint32))
    assert not raw[payload:].any()
    back = [torch.full((n,), float("nan")) for _ in range(3)]
    read_unit_opts(str(tmp_path), 4, back, share=share, rank=1)
    for a, b in zip(blocks, back):
        assert np.array_equal(a.numpy().view(np.uint32), b.numpy().view(np.uint32))


def test_empty_share_has_no_file_and_mismatches_are_errors(tmp_path):
    empty = [torch.empty(0) for _ in range(3)]
    assert write_unit_opts(str(tmp_path), 0, empty) is None
    assert os.listdir(tmp_path) == []
    read_unit_opts(str(tmp_path), 0, empty)  # nothing to read, no file needed
    blocks = [torch.zeros(100) for _ in range(3)]
    write_unit_opts(str(tmp_path), 0, blocks, share=FORWARD_SHARE)
    with pytest.raises(ValueError, match="bytes on disk"):
        read_unit_opts(str(tmp_path), 0, [torch.zeros(101) for _ in range(3)], share=FORWARD_SHARE)
    with pytest.raises(ValueError, match="equal length"):
        write_unit_opts(str(tmp_path), 0, [torch.zeros(4), torch.zeros(5), torch.zeros(4)])
    with pytest.raises(FileNotFoundError):
        read_unit_opts(str(tmp_path), 9, blocks)
    with pytest.raises(ValueError, match="contiguous host"):
        write_unit_opts(str(tmp_path), 0, [torch.zeros(8)[::2] for _ in range(3)])
