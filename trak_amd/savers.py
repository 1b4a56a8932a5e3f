"""On-disk store of TRAK results in the layout of the reference's `MmapSaver`
(trak/savers.py:241-457), so that a `save_dir` written here can be resumed by a stock TRAKer
and the other way round.  `TRAKer(saver=trak_amd.MmapSaver)` takes the class
(trak/traker.py:201-211).

Layout of `save_dir` (every `.mmap` file is a `.npy`-format array created with
`numpy.lib.format.open_memmap`, element type float16 or float32 depending on
`use_half_precision` unless noted):

    metadata.json                       {"JL dimension", "JL matrix type", "train set size"}
    experiments.json                    {exp_name: {"num_targets", "scores_path", "scores_finalized"}}
    id_<model_id>.json                  {"<model_id>": {"is_featurized", "is_finalized"}}
    <model_id>/grads.mmap               [train_set_size, proj_dim]
    <model_id>/out_to_loss.mmap         [train_set_size, 1]
    <model_id>/features.mmap            [train_set_size, proj_dim]
    <model_id>/_is_featurized.mmap      [train_set_size, 1] int32
    <model_id>/<exp_name>_grads.mmap    [num_targets, proj_dim]
    scores/<exp_name>.mmap              [train_set_size, num_targets]
"""
import json
import logging
import os
from abc import ABC, abstractmethod
from pathlib import Path

import numpy as np
from numpy.lib.format import open_memmap

_METADATA_KEYS = ("JL dimension", "JL matrix type", "train set size")


class ModelIDException(Exception):
    """Raised for a model ID that is registered twice or whose folder is missing
    (trak/savers.py:235-238)."""


def _read_json(path):
    with open(path, "r") as f:
        return json.load(f)


def _write_json(path, content):
    with open(path, "w") as f:
        json.dump(content, f)


class AbstractSaver(ABC):
    """Metadata handling shared by savers (trak/savers.py:22-232): creates `save_dir`, checks the
    run's hyperparameters against `metadata.json`, and reads the model IDs and experiments that
    are already there."""

    @abstractmethod
    def __init__(self, save_dir, metadata, load_from_save_dir, logging_level, use_half_precision) -> None:
        self.metadata = metadata
        self.save_dir = Path(save_dir).resolve()
        self.load_from_save_dir = load_from_save_dir
        self.use_half_precision = use_half_precision

        os.makedirs(self.save_dir.joinpath("scores"), exist_ok=True)
        self.logger = logging.getLogger("STORE")
        self.logger.setLevel(logging_level)

        self.metadata_file = self.save_dir.joinpath("metadata.json")
        self.experiments_file = self.save_dir.joinpath("experiments.json")
        self.model_ids = {}
        self.experiments = {}
        if self.load_from_save_dir:
            self._check_or_write_metadata()
            self._read_existing()
        self._log_existing()

        self.current_model_id = None
        self.current_store = {"grads": None, "out_to_loss": None, "features": None}

    def _check_or_write_metadata(self):
        if not os.path.exists(self.metadata_file):
            _write_json(self.metadata_file, self.metadata)
            return
        on_disk = _read_json(self.metadata_file)
        found = int(on_disk["JL dimension"])
        assert self.metadata["JL dimension"] == found, (
            f"In {self.save_dir} there are models using JL dimension {found},\n"
            f"and this TRAKer instance uses JL dimension {self.metadata['JL dimension']}."
        )
        found = on_disk["JL matrix type"]
        assert self.metadata["JL matrix type"] == found, (
            f"In {self.save_dir} there are models using a {found} JL matrix,\n"
            f"and this TRAKer instance uses a {self.metadata['JL matrix type']} JL matrix."
        )
        found = on_disk["train set size"]
        assert self.metadata["train set size"] == found, (
            f"In {self.save_dir} there are models TRAKing\n{found} examples, and in this TRAKer instance\n"
            f"there are {self.metadata['train set size']} examples."
        )

    def _read_existing(self):
        for id_file in self.save_dir.rglob("id_*.json"):
            for model_id, state in _read_json(id_file).items():
                self.model_ids[int(model_id)] = state
        if os.path.isfile(self.experiments_file):
            self.experiments.update(_read_json(self.experiments_file))
        else:
            _write_json(self.experiments_file, {})

    def _log_existing(self):
        ids = sorted(self.model_ids)
        if ids:
            self.logger.info(f"Existing model IDs in {self.save_dir}: {ids}")
            done = [i for i in ids if self.model_ids[i]["is_finalized"] == 1]
            if done:
                self.logger.info(f"Model IDs that have been finalized: {done}")
            else:
                self.logger.info(f"No model IDs in {self.save_dir} have been finalized.")
        else:
            self.logger.info(f"No existing model IDs in {self.save_dir}.")
        if self.experiments:
            self.logger.info("Existing TRAK scores:")
            for exp_name, values in self.experiments.items():
                self.logger.info(f"{exp_name}: {values['scores_path']}")
        else:
            self.logger.info(f"No existing TRAK scores in {self.save_dir}.")

    @abstractmethod
    def register_model_id(self, model_id: int) -> None:
        """Creates the metadata and the store of a new model ID (checkpoint)."""

    @abstractmethod
    def serialize_current_model_id_metadata(self) -> None:
        """Commits the state of the current model ID to disk."""

    @abstractmethod
    def init_store(self, model_id: int) -> None:
        """Creates the store of a model ID."""

    @abstractmethod
    def init_experiment(self, model_id: int) -> None:
        """Creates the store of an experiment (a set of targets) for a model ID."""

    @abstractmethod
    def load_current_store(self, model_id: int) -> None:
        """Points `current_store` at the arrays of a model ID."""

    @abstractmethod
    def save_scores(self, exp_name: str) -> None:
        """Commits the scores of an experiment."""

    @abstractmethod
    def del_grads(self, model_id: int, target: bool) -> None:
        """Deletes the projected gradients of a model ID."""


class MmapSaver(AbstractSaver):
    """Saver on memory-mapped `.npy` files (trak/savers.py:241-457): small reads and writes while
    featurizing touch only the pages they need."""

    def __init__(
        self,
        save_dir,
        metadata,
        train_set_size,
        proj_dim,
        load_from_save_dir,
        logging_level,
        use_half_precision,
    ) -> None:
        super().__init__(
            save_dir=save_dir,
            metadata=metadata,
            load_from_save_dir=load_from_save_dir,
            logging_level=logging_level,
            use_half_precision=use_half_precision,
        )
        self.train_set_size = train_set_size
        self.proj_dim = proj_dim

    # -- model IDs ---------------------------------------------------------------------------

    def _model_dir(self, model_id):
        return self.save_dir.joinpath(str(model_id))

    def register_model_id(self, model_id: int, _allow_featurizing_already_registered: bool) -> None:
        """Raises ModelIDException when the ID exists (unless re-featurizing is allowed), otherwise
        creates its arrays and its `id_<model_id>.json` (trak/savers.py:268-295)."""
        self.current_model_id = model_id
        if model_id in self.model_ids and not _allow_featurizing_already_registered:
            raise ModelIDException(f"model id {model_id} is already registered. Check {self.save_dir}")
        self.model_ids[model_id] = {"is_featurized": 0, "is_finalized": 0}
        self.init_store(model_id)
        self.serialize_current_model_id_metadata(already_exists=False)

    def serialize_current_model_id_metadata(self, already_exists=True) -> None:
        """`is_featurized` becomes 1 once every training example is marked; the JSON file is
        (re)written on registration and when that happens (trak/savers.py:297-315)."""
        model_id = self.current_model_id
        done = int(self.current_store["is_featurized"].sum() == self.train_set_size)
        self.model_ids[model_id]["is_featurized"] = done
        if done == 1 or not already_exists:
            state = {"is_featurized": done, "is_finalized": self.model_ids[model_id]["is_finalized"]}
            _write_json(self.save_dir.joinpath(f"id_{model_id}.json"), {model_id: state})

    def init_store(self, model_id) -> None:
        """Creates (or truncates) the four arrays of a model ID, zero filled
        (trak/savers.py:317-332)."""
        prefix = self._model_dir(model_id)
        if os.path.exists(prefix):
            self.logger.info(f"Model ID folder {prefix} already exists")
        os.makedirs(prefix, exist_ok=True)
        self.load_current_store(model_id, mode="w+")

    # -- experiments -------------------------------------------------------------------------

    def init_experiment(self, exp_name, num_targets, model_id) -> None:
        """Registers the experiment in `experiments.json` and opens (or creates) its target
        gradients for this model ID and its scores (trak/savers.py:334-361)."""
        prefix = self._model_dir(model_id)
        if not os.path.exists(prefix):
            raise ModelIDException(f"model ID folder {prefix} does not exist,\ncannot start scoring")
        self.experiments[exp_name] = {
            "num_targets": num_targets,
            "scores_path": str(self.save_dir.joinpath(f"scores/{exp_name}.mmap")),
            "scores_finalized": 0,
        }
        on_disk = _read_json(self.experiments_file)
        on_disk[exp_name] = self.experiments[exp_name]
        _write_json(self.experiments_file, on_disk)

        mode = "r+" if os.path.exists(prefix.joinpath(f"{exp_name}_grads.mmap")) else "w+"
        self.load_current_store(model_id=model_id, exp_name=exp_name, exp_num_targets=num_targets, mode=mode)

    # -- arrays ------------------------------------------------------------------------------

    def _load(self, fname, shape, mode, dtype=None):
        """`.npy`-format memmap; a missing file in a read mode gives None
        (trak/savers.py:363-374)."""
        self.logger.debug(f"{'Creating' if mode == 'w+' else 'Loading'} {fname}.")
        if dtype is None:
            dtype = np.float16 if self.use_half_precision else np.float32
        try:
            return open_memmap(filename=fname, mode=mode, shape=shape, dtype=dtype)
        except OSError:
            self.logger.info(f"{fname} does not exist, skipping.")
            return None

    def load_current_store(self, model_id, exp_name=None, exp_num_targets=-1, mode="r+") -> None:
        """Opens the arrays of a model ID (exp_name None) or of one of its experiments into
        `current_store` (trak/savers.py:376-442)."""
        self.current_model_id = model_id
        prefix = self._model_dir(model_id)
        N, k = self.train_set_size, self.proj_dim
        if exp_name is None:
            wanted = [
                ("grads", prefix.joinpath("grads.mmap"), (N, k), None),
                ("out_to_loss", prefix.joinpath("out_to_loss.mmap"), (N, 1), None),
                ("features", prefix.joinpath("features.mmap"), (N, k), None),
                ("is_featurized", prefix.joinpath("_is_featurized.mmap"), (N, 1), np.int32),
            ]
        else:
            self.current_experiment_name = exp_name
            wanted = [
                (f"{exp_name}_grads", prefix.joinpath(f"{exp_name}_grads.mmap"), (exp_num_targets, k), None),
                (f"{exp_name}_scores", self.save_dir.joinpath(f"scores/{exp_name}.mmap"), (N, exp_num_targets), None),
            ]
        for name, path, shape, dtype in wanted:
            self.current_store[name] = self._load(path, shape, mode, dtype)

    def save_scores(self, exp_name):
        """Flushes the scores and marks the experiment finalized (trak/savers.py:444-451)."""
        assert self.current_experiment_name == exp_name
        self.logger.info(f"Saving scores in {self.save_dir.joinpath('scores')}/{exp_name}.mmap")
        self.current_store[f"{exp_name}_scores"].flush()
        self.experiments[exp_name]["scores_finalized"] = 1
        _write_json(self.experiments_file, self.experiments)

    def del_grads(self, model_id):
        """Removes `grads.mmap` of a model ID (trak/savers.py:453-457)."""
        self._model_dir(model_id).joinpath("grads.mmap").unlink()
