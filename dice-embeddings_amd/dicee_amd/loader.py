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


def save_experiment(path, model, entity_to_idx, relation_to_idx, extra_config=None):
    """Write ``model`` and its vocabularies in dicee's on-disk layout (used by tests and examples)."""
    os.makedirs(path, exist_ok=True)
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
