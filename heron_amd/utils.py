"""Small helpers shared across the package (naming, encoding, directories).

``genKey``, ``Code``/``DeCode``, ``anaCostModel`` and ``mkdir`` keep the behaviour of the
reference's utils.py:21-39, 306-332, 55-62.
"""
import os
import random
import shutil


def genKey(type_, stage_name=None, ax_name=None, param_name=None, var_name=None, others=None):
    """Names of CSP variables: L# loop extents, P# tunable parameters, V# derived values, O# auxiliaries."""
    assert type_ in ["L", "P", "V", "O"]
    if type_ == "L":
        assert ax_name and stage_name
        return type_ + "#" + "ST:%s,AX:%s" % (stage_name, ax_name)
    elif type_ == "P":
        assert param_name
        return type_ + "#" + "ST:%s,AX:%s,PA:%s" % (stage_name, ax_name, param_name)
    elif type_ == "V":
        assert var_name
        return type_ + "#" + "ST:%s,AX:%s,VA:%s" % (stage_name, ax_name, var_name)
    assert others
    return type_ + "#" + "ST:%s,AX:%s,OT:%s" % (stage_name, ax_name, others)


def mkdir(name):
    if not os.path.exists(name):
        print("%s not exists, create one" % name)
        os.makedirs(name)
    else:
        print("%s exists, remove and create one" % name)
        shutil.rmtree(name)
        os.makedirs(name)


def Code(point):
    assert isinstance(point, list)
    return ''.join(str(x) + '_' for x in point)


def DeCode(code):
    assert isinstance(code, str)
    return [int(x) for x in code.split('_')[:-1]]


def anaCostModel(model, key_list):
    """Variable names ordered by the cost model's feature importance (random when untrained)."""
    bst = model.bst
    if bst is None:
        random.shuffle(key_list)
        return key_list
    score_map = bst.get_score(importance_type='weight')
    score_list_sorted = sorted(score_map.items(), key=lambda x: -x[1])
    selected_idxs = [int(x[0].split('f')[1]) for x in score_list_sorted]
    missing = [x for x in range(len(key_list)) if x not in selected_idxs]
    return [key_list[x] for x in selected_idxs + missing]


def removedot(name):
    if isinstance(name, str):
        return name.replace('.', '_')
    return name
