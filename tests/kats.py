"""Known-answer data of the reference's own tests, loaded from tests/golden/reference_kats.json
(expectations only; see the "_source" entry there for the file:line of each).

Trees are nested (n_seqs, tokens, [children]) tuples; tails are child-index paths from the root.
"""
import json
import os

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_kats.json")) as _f:
    _D = json.load(_f)


def _tree(j):
    return (j["n_seqs"], tuple(j["tokens"]), [_tree(c) for c in j["children"]])


ADD_SEQ_STEPS = [(s["tokens"], _tree(s["tree"]), [tuple(p) for p in s["tails"]]) for s in _D["add_seq_steps"]]
ADD_SEQ_INDICES = _D["add_seq_returned_indices"]
APPEND_CASE = {"adds": _D["append_case"]["adds"], "append": _D["append_case"]["append"],
               "tree": _tree(_D["append_case"]["tree"]), "tails": [tuple(p) for p in _D["append_case"]["tails"]]}
REMOVE_CASE = {"adds": _D["remove_case"]["adds"], "remove": _D["remove_case"]["remove"],
               "tree": _tree(_D["remove_case"]["tree"])}
TABLE_KAT = dict(_D["table_kat"])
TABLE_KAT["rows"] = [(tuple(r[0]), r[1], r[2]) for r in _D["table_kat"]["rows"]]
