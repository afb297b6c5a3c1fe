"""MI355X-native KvsAll scoring, filtered-rank evaluation and top-k prediction for dicee-style
knowledge-graph-embedding models (DistMult, ComplEx, QMult, OMult, Keci).

The compute path is a hand-written HIP library (``libkge_hip.so``, C ABI in ``include/kge_hip.h``);
this package is the thin Python side that mirrors the reference's call surface:

* ``models``     ``DistMult/ComplEx/QMult/OMult/Keci/CKeci`` with ``forward``, ``forward_k_vs_all``,
                 ``k_vs_all_score`` (dicee/models/*.py)
* ``evaluator``  ``Evaluator.evaluate_lp_k_vs_all`` (dicee/evaluation/evaluator.py:394-510)
* ``link_prediction``  ``evaluate_lp``: head and tail direction (dicee/evaluation/link_prediction.py:351-473)
* ``ensemble``   ``evaluate_ensemble_link_prediction_performance`` (dicee/evaluation/ensemble.py:20-135)
* ``kge``        ``KGE.predict_topk`` / ``predict`` / ``predict_missing_tail_entity``
                 (dicee/knowledge_graph_embeddings.py:314-579)
* ``csr``        the known-answer filter as a CSR (dicee's ``er_vocab``)
* ``loader``     ``load_model`` / ``load_splits`` / ``evaluate_experiment`` for a dicee experiment folder
                 (dicee/static_funcs.py:246-299, read_preprocess_save_load_kg/save_load_disk.py:40-44)
* ``ops``        tensor-level wrappers of the C ABI

There is no CPU fallback: every scoring call raises if the HIP library is not built or no GPU is
present.
"""
from . import _lib  # noqa: F401
from .csr import FilterCSR  # noqa: F401
from .models import DistMult, ComplEx, QMult, OMult, Keci, CKeci, MODEL_REGISTRY, initialize_model  # noqa: F401
from .evaluator import Evaluator, compute_metrics_from_ranks_simple  # noqa: F401
from .kge import KGE  # noqa: F401
from .ensemble import evaluate_ensemble_link_prediction_performance  # noqa: F401
from .link_prediction import (evaluate_lp, evaluate_link_prediction_performance,  # noqa: F401
                              evaluate_link_prediction_performance_with_reciprocals)
from .loader import load_model, load_splits, evaluate_experiment, save_experiment  # noqa: F401

__version__ = "0.1.0"
