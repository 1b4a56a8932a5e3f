"""trak_amd.MmapSaver against the on-disk snapshot of the reference's own MmapSaver
(tests/golden/saver_layout.json, written by tests/golden/make_saver_layout.py from
trak/savers.py:241-457) and its error behaviour."""
import json
import logging
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import saver_scenario  # noqa: E402

from trak_amd.savers import AbstractSaver, MmapSaver, ModelIDException  # noqa: E402

with open(os.path.join(HERE, "golden", "saver_layout.json")) as f:
    GOLDEN = json.load(f)


@pytest.mark.parametrize("half", [False, True])
def test_directory_equals_reference_snapshot(tmp_path, half):
    reopened = saver_scenario.run(MmapSaver, str(tmp_path), use_half_precision=half)
    want = GOLDEN["float16" if half else "float32"]
    got = saver_scenario.snapshot(str(tmp_path))
    assert sorted(got) == sorted(want["files"])
    for rel in want["files"]:
        assert got[rel] == want["files"][rel], rel
    assert reopened == want["reopened"]


def _kw(tmp_path, **over):
    kw = dict(
        save_dir=str(tmp_path), metadata={"JL dimension": 8, "JL matrix type": "rademacher", "train set size": 12},
        train_set_size=12, proj_dim=8, load_from_save_dir=True, logging_level=logging.ERROR, use_half_precision=False,
    )
    kw.update(over)
    return kw


def test_is_a_saver_class_for_traker(tmp_path):
    # TRAKer instantiates `saver(save_dir=, metadata=, train_set_size=, proj_dim=, load_from_save_dir=,
    # logging_level=, use_half_precision=)` (trak/traker.py:203-211)
    s = MmapSaver(**_kw(tmp_path))
    assert isinstance(s, AbstractSaver)
    assert s.current_model_id is None
    assert s.current_store == {"grads": None, "out_to_loss": None, "features": None}
    assert os.path.isdir(tmp_path / "scores")
    assert json.load(open(tmp_path / "metadata.json"))["JL dimension"] == 8
    assert json.load(open(tmp_path / "experiments.json")) == {}


def test_metadata_mismatch_asserts(tmp_path):
    MmapSaver(**_kw(tmp_path))
    for key, value in (("JL dimension", 16), ("JL matrix type", "normal"), ("train set size", 13)):
        meta = {"JL dimension": 8, "JL matrix type": "rademacher", "train set size": 12}
        meta[key] = value
        with pytest.raises(AssertionError):
            MmapSaver(**_kw(tmp_path, metadata=meta))


def test_no_load_from_save_dir_touches_no_metadata(tmp_path):
    s = MmapSaver(**_kw(tmp_path, load_from_save_dir=False))
    assert not os.path.exists(tmp_path / "metadata.json")
    assert not os.path.exists(tmp_path / "experiments.json")
    assert s.model_ids == {} and s.experiments == {}


def test_duplicate_model_id_and_missing_folder(tmp_path):
    s = MmapSaver(**_kw(tmp_path))
    s.register_model_id(1, _allow_featurizing_already_registered=False)
    with pytest.raises(ModelIDException):
        s.register_model_id(1, _allow_featurizing_already_registered=False)
    s.register_model_id(1, _allow_featurizing_already_registered=True)  # allowed: store re-created
    assert int(s.current_store["is_featurized"].sum()) == 0
    with pytest.raises(ModelIDException):
        s.init_experiment("e", 3, model_id=9)


def test_store_shapes_dtypes_and_resume(tmp_path):
    s = MmapSaver(**_kw(tmp_path, use_half_precision=True))
    s.register_model_id(0, _allow_featurizing_already_registered=False)
    st = s.current_store
    assert st["grads"].shape == (12, 8) and st["grads"].dtype == np.float16
    assert st["out_to_loss"].shape == (12, 1) and st["features"].shape == (12, 8)
    assert st["is_featurized"].shape == (12, 1) and st["is_featurized"].dtype == np.int32
    st["grads"][3] = 2.0
    st["is_featurized"][3] = 1
    s.serialize_current_model_id_metadata()
    st["grads"].flush()
    st["is_featurized"].flush()
    # a fresh instance sees the partial state (trak/traker.py:416-423 skips rows already done)
    s2 = MmapSaver(**_kw(tmp_path, use_half_precision=True))
    assert s2.model_ids == {0: {"is_featurized": 0, "is_finalized": 0}}
    s2.load_current_store(0)
    assert float(s2.current_store["grads"][3, 0]) == 2.0
    assert int(s2.current_store["is_featurized"].sum()) == 1
    # experiment arrays; loading an experiment that was never created gives None entries
    s2.init_experiment("q", 4, 0)
    assert s2.current_store["q_grads"].shape == (4, 8)
    assert s2.current_store["q_scores"].shape == (12, 4)
    s2.load_current_store(0, "never", 4)
    assert s2.current_store["never_grads"] is None
    with pytest.raises(AssertionError):
        s2.save_scores("q")  # the current experiment is "never"
    s2.load_current_store(0, "q", 4)
    s2.save_scores("q")
    assert json.load(open(tmp_path / "experiments.json"))["q"]["scores_finalized"] == 1
    s2.del_grads(0)
    assert not os.path.exists(tmp_path / "0" / "grads.mmap")


def test_files_open_with_plain_numpy(tmp_path):
    s = MmapSaver(**_kw(tmp_path))
    s.register_model_id(5, _allow_featurizing_already_registered=False)
    s.current_store["grads"][:] = np.arange(96, dtype=np.float32).reshape(12, 8)
    s.current_store["grads"].flush()
    a = np.load(tmp_path / "5" / "grads.mmap", mmap_mode="r")
    assert a.shape == (12, 8) and a.dtype == np.float32 and float(a[11, 7]) == 95.0
