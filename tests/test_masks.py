"""Host logic next to the hot path: mask file format and the dense-to-sparse transition test (CPU only)."""
import pickle

import pytest
import torch

from spion_amd import TransitionDetector, load_mask_list, save_mask_list, stack_for_replicas


def test_mask_file_round_trip_and_reference_format(tmp_path):
    layers = [(torch.rand(8, 8) > 0.7).float() for _ in range(2)]
    mat_lst = stack_for_replicas(layers)
    assert mat_lst.shape == (4, 2, 8, 8) and torch.equal(mat_lst[0], mat_lst[3])
    path = tmp_path / "mat_lst_lra-image_test.pickle"
    save_mask_list(mat_lst, str(path))
    # what the reference's reader does with the file (main_inference.py:164-166) -- on a file this test wrote
    with open(path, "rb") as f:
        plain = pickle.load(f)
    assert isinstance(plain, torch.Tensor) and torch.equal(plain, mat_lst)
    # and a file written the reference's way (main_conv_ff.py:305-306) loads through the restricted reader
    path2 = tmp_path / "written_like_the_reference.pickle"
    with open(path2, "wb") as f:
        pickle.dump(mat_lst, f, pickle.HIGHEST_PROTOCOL)
    got = load_mask_list(str(path2))
    assert got.dtype == torch.float32 and torch.equal(got, mat_lst)


def test_mask_file_reader_refuses_other_content(tmp_path):
    path = tmp_path / "evil.pickle"
    with open(path, "wb") as f:
        pickle.dump({"fn": print}, f)
    with pytest.raises(pickle.UnpicklingError):
        load_mask_list(str(path))
    path2 = tmp_path / "wrong_shape.pickle"
    with open(path2, "wb") as f:
        pickle.dump(torch.zeros(3, 3), f)
    with pytest.raises(ValueError):
        load_mask_list(str(path2))


def _maps(*values):
    return [torch.tensor([[float(v)]]) for v in values]


def test_transition_detector_hand_worked_sequences():
    # one layer, 1x1 "maps": distances are absolute differences
    det = TransitionDetector(1)
    assert det.update(_maps(0.0)) is False          # first evaluation: stored
    assert det.update(_maps(10.0)) is False         # second: distance 10 recorded, reference map stays at 0
    assert det.update(_maps(10.5)) is True          # third: distance to the FIRST map 10.5, change 5 % < 15 %
    assert det.update(_maps(99.0)) is True          # stays settled

    det = TransitionDetector(1)
    det.update(_maps(0.0))
    det.update(_maps(10.0))
    assert det.update(_maps(20.0)) is False         # distance 20, change 100 %: reference map becomes 20
    assert det.update(_maps(41.0)) is True          # distance 21, change 5 %


def test_transition_detector_truncates_and_needs_every_layer():
    det = TransitionDetector(1)
    det.update(_maps(0.0))
    det.update(_maps(100.0))
    assert det.update(_maps(115.9)) is False        # 15.9 % truncates to 15: not below 15
    det = TransitionDetector(1)
    det.update(_maps(0.0))
    det.update(_maps(100.0))
    assert det.update(_maps(114.99)) is True        # 14.99 % truncates to 14
    det = TransitionDetector(2)
    det.update(_maps(0.0, 0.0))
    det.update(_maps(10.0, 10.0))
    assert det.update(_maps(10.5, 30.0)) is False   # layer 1 changed by 200 %
    assert abs(det.diff[0] - 5.0) < 1e-4 and abs(det.diff[1] - 200.0) < 1e-3


def test_transition_detector_identical_maps_do_not_settle():
    # two identical maps in a row: the previous distance is 0 and the change is 0/0 or x/0; the layer is not settled
    det = TransitionDetector(1)
    det.update(_maps(5.0))
    assert det.update(_maps(5.0)) is False          # distance 0 recorded
    assert det.update(_maps(5.0)) is False          # 0/0: not settled, the kept map is replaced
    assert det.update(_maps(7.0)) is False          # 2/0 = inf: not settled
    assert det.update(_maps(9.0)) is True           # distance 2 after 2: change 0 %
