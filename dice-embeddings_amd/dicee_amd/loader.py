"""Read (and, for tests, write) a dicee experiment folder.

A trained dicee run leaves ``model.pt`` (a ``state_dict``), ``configuration.json`` (the training
arguments), ``report.json`` (``num_entities``, ``num_relations``, ...) and the index files
``entity_to_idx.csv`` / ``relation_to_idx.csv`` (one column ``entity`` / ``relation``, row number =
id).  ``load_model`` mirrors dicee.static_funcs.load_model (dicee/static_funcs.py:246-299) for the
four model families this build accelerates; nothing is unpickled: ``model.pt`` is read with
``torch.load(..., weights_only=True)``.
"""
import csv
import json
import os

import numpy as np
import torch

from .models import MODEL_REGISTRY, initialize_model


def _read_index_csv(path, column):
    out = {}
    with open(path, newline="", encoding="utf-8") as f:
        reader = csv.reader(f)
        header = next(reader)
        col = header.index(column)
        for row in reader:
            if row:
                out[row[col]] = int(row[0])
    return out


def load_json(path):
    with open(path, "r") as f:
        return json.load(f)


def load_model(path_of_experiment_folder, model_name="model.pt", device=None):
    """(model, (entity_to_idx, relation_to_idx)); parameters frozen, eval mode, moved to ``device``."""
    if not os.path.isdir(path_of_experiment_folder):
        raise AssertionError(f"Could not find a directory {path_of_experiment_folder}")
    configs = load_json(os.path.join(path_of_experiment_folder, "configuration.json"))
    reports = load_json(os.path.join(path_of_experiment_folder, "report.json"))
    if configs.get("byte_pair_encoding", None):
        raise NotImplementedError("byte-pair-encoded models are outside the accelerated path")
    if configs.get("model") not in MODEL_REGISTRY:
        raise ValueError(f"--model_name: {configs.get('model')} is not found.")
    configs["num_entities"] = reports["num_entities"]
    configs["num_relations"] = reports["num_relations"]
    weights = torch.load(os.path.join(path_of_experiment_folder, model_name), map_location="cpu", weights_only=True)
    model, _ = initialize_model(configs)
    model.load_state_dict(weights)
    for parameter in model.parameters():
        parameter.requires_grad = False
    model.eval()
    if device is not None:
        model = model.to(device)
    entity_to_idx = _read_index_csv(os.path.join(path_of_experiment_folder, "entity_to_idx.csv"), "entity")
    relation_to_idx = _read_index_csv(os.path.join(path_of_experiment_folder, "relation_to_idx.csv"), "relation")
    assert sorted(entity_to_idx.values()) == list(range(len(entity_to_idx)))
    assert sorted(relation_to_idx.values()) == list(range(len(relation_to_idx)))
    return model, (entity_to_idx, relation_to_idx)


def load_splits(path_of_experiment_folder):
    """``{'train_set': ndarray[n,3], 'valid_set': ..., 'test_set': ...}`` from the ``*_set.npy`` files a dicee run
    leaves next to its model (dicee/read_preprocess_save_load_kg/save_load_disk.py:40-44; integer ids in the
    narrowest type that holds them, dicee/static_funcs.py:373-392).  Missing splits are ``None``."""
    out = {}
    for name in ("train_set", "valid_set", "test_set"):
        f = os.path.join(path_of_experiment_folder, name + ".npy")
        out[name] = np.load(f, allow_pickle=False) if os.path.isfile(f) else None
    if out["train_set"] is None:
        raise FileNotFoundError(os.path.join(path_of_experiment_folder, "train_set.npy"))
    return out


def evaluate_experiment(path_of_experiment_folder, eval_model="train_val_test", batch_size=None, device="cuda",
                        tie="stable"):
    """Filtered link-prediction report of a stored dicee run: model and id triples from the folder, the filter
    vocabulary built on the GPU over all stored splits, one fused rank call per batch.  Returns the dict the
    reference writes to ``eval_report.json`` (``{'Train': {'H@1', 'H@3', 'H@10', 'MRR'}, 'Val': ..., 'Test': ...}``)."""
    from types import SimpleNamespace
    from .evaluator import Evaluator
    model, _ = load_model(path_of_experiment_folder, device=device)
    splits = load_splits(path_of_experiment_folder)
    configs = load_json(os.path.join(path_of_experiment_folder, "configuration.json"))
    args = SimpleNamespace(batch_size=int(batch_size or configs.get("batch_size") or 1024), eval_model=eval_model,
                           scoring_technique="KvsAll", full_storage_path=None)
    dataset = SimpleNamespace(num_entities=model.num_entities, num_relations=model.num_relations, er_vocab=None,
                              **splits)
    evaluator = Evaluator(args, tie=tie)
    report = evaluator.eval(dataset, model, "EntityPrediction", during_training=True)
    return report, evaluator


def save_experiment(path, model, entity_to_idx, relation_to_idx, extra_config=None, splits=None):
    """Write ``model`` and its vocabularies in dicee's on-disk layout (used by tests and examples)."""
    os.makedirs(path, exist_ok=True)
    for name, triples in (splits or {}).items():
        if triples is not None:
            np.save(os.path.join(path, name + ".npy"), np.asarray(triples))
    torch.save({k: v.detach().cpu() for k, v in model.state_dict().items()}, os.path.join(path, "model.pt"))
    cfg = {k: v for k, v in model.args.items() if isinstance(v, (int, float, str, bool, type(None)))}
    cfg["model"] = model.name
    cfg.update(extra_config or {})
    with open(os.path.join(path, "configuration.json"), "w") as f:
        json.dump(cfg, f, indent=2)
    with open(os.path.join(path, "report.json"), "w") as f:
        json.dump({"num_entities": model.num_entities, "num_relations": model.num_relations}, f)
    for fname, column, vocab in (("entity_to_idx.csv", "entity", entity_to_idx),
                                 ("relation_to_idx.csv", "relation", relation_to_idx)):
        with open(os.path.join(path, fname), "w", newline="", encoding="utf-8") as f:
            w = csv.writer(f)
            w.writerow(["", column])
            for name, idx in sorted(vocab.items(), key=lambda kv: kv[1]):
                w.writerow([idx, name])
