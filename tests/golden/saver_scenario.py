"""A fixed sequence of saver calls (the ones TRAKer makes while featurizing, finalizing and scoring)
and a snapshot of the directory they leave behind.  Applied to the reference's MmapSaver by
make_saver_layout.py (which writes saver_layout.json) and to this package's MmapSaver by the tests:
the two snapshots must be equal."""
import hashlib
import json
import logging
import os

import numpy as np

TRAIN, PROJ, TARGETS = 12, 8, 5


def run(saver_cls, save_dir, use_half_precision, matrix_type="rademacher"):
    """Returns what a second saver instance, opened on the finished directory, reports."""
    metadata = {"JL dimension": PROJ, "JL matrix type": matrix_type, "train set size": TRAIN}
    kw = dict(
        save_dir=save_dir, metadata=metadata, train_set_size=TRAIN, proj_dim=PROJ, load_from_save_dir=True,
        logging_level=logging.ERROR, use_half_precision=use_half_precision,
    )
    rng = np.random.default_rng(7)
    s = saver_cls(**kw)
    s.register_model_id(0, _allow_featurizing_already_registered=False)
    # featurize in two batches (trak/traker.py:425-437)
    for inds in (np.arange(0, 7), np.arange(7, TRAIN)):
        s.current_store["grads"][inds] = rng.standard_normal((len(inds), PROJ)).astype(np.float32)
        s.current_store["out_to_loss"][inds] = rng.random((len(inds), 1)).astype(np.float32)
        s.current_store["is_featurized"][inds] = 1
        s.serialize_current_model_id_metadata()
    # finalize_features (trak/traker.py:480-491)
    s.load_current_store(0)
    s.current_store["features"][:] = np.asarray(s.current_store["grads"]) * 0.5
    s.model_ids[0]["is_finalized"] = 1
    s.serialize_current_model_id_metadata()
    # a second, partly featurized model
    s.register_model_id(3, _allow_featurizing_already_registered=False)
    s.current_store["grads"][np.arange(4)] = rng.standard_normal((4, PROJ)).astype(np.float32)
    s.current_store["is_featurized"][np.arange(4)] = 1
    s.serialize_current_model_id_metadata()
    # scoring (trak/traker.py:518, :576, :630-681)
    s.init_experiment("exp", TARGETS, 0)
    s.current_store["exp_grads"][np.arange(TARGETS)] = rng.standard_normal((TARGETS, PROJ)).astype(np.float32)
    s.load_current_store(0, "exp", TARGETS)
    s.current_store["exp_scores"][:] = rng.standard_normal((TRAIN, TARGETS)).astype(np.float32)
    s.save_scores("exp")
    s.del_grads(0)
    for v in s.current_store.values():
        if v is not None:
            v.flush()
    again = saver_cls(**kw)
    return {
        "model_ids": {str(k): v for k, v in sorted(again.model_ids.items())},
        "experiments": _strip(again.experiments, save_dir),
    }


def _strip(obj, save_dir):
    """JSON content with the absolute directory replaced by a placeholder."""
    text = json.dumps(obj, sort_keys=True)
    return json.loads(text.replace(str(os.path.realpath(save_dir)), "<save_dir>"))


def snapshot(save_dir):
    """{relative path: description}: parsed JSON for .json files; for .mmap files the raw `.npy`
    header, the file size and a digest of the data."""
    out = {}
    for root, _, files in os.walk(save_dir):
        for name in sorted(files):
            path = os.path.join(root, name)
            rel = os.path.relpath(path, save_dir)
            if name.endswith(".json"):
                with open(path) as f:
                    out[rel] = _strip(json.load(f), save_dir)
            else:
                with open(path, "rb") as f:
                    raw = f.read()
                assert raw[:6] == b"\x93NUMPY"
                hlen = int.from_bytes(raw[8:10], "little") if raw[6] == 1 else int.from_bytes(raw[8:12], "little")
                start = (10 if raw[6] == 1 else 12) + hlen
                out[rel] = {
                    "header": raw[:start].decode("latin1"),
                    "size": len(raw),
                    "sha256": hashlib.sha256(raw[start:]).hexdigest(),
                }
    return dict(sorted(out.items()))
