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
    """The variable names of ``key_list`` ordered by how much the cost model relies on each (feature ``f<i>`` of the
    booster is variable ``i``); variables the trees never split on keep their order behind the ranked ones.  An
    untrained model ranks nothing: the list is shuffled in place and returned.  Same contract as utils.py:319-332 of
    the reference."""
    if model.bst is None:
        random.shuffle(key_list)
        return key_list
    weight = [0.0] * len(key_list)
    for name, score in model.bst.get_score(importance_type='weight').items():
        idx = int(name[1:])
        if 0 <= idx < len(weight):
            weight[idx] = float(score)
    order = sorted(range(len(key_list)), key=lambda i: (weight[i] <= 0.0, -weight[i], i))
    return [key_list[i] for i in order]


def removedot(name):
    if isinstance(name, str):
        return name.replace('.', '_')
    return name
