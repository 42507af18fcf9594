"""Tuning configuration.  Field names, defaults and the JSON schema of a case file are the reference's
(config.py:4-54): ``{"config": {"out_name", "method", "max_trials", "runner_number", "runner_repeat",
"runner_timeout", "build_timeout", "in_dtype", "out_dtype", "cases": {name: [op, shape]}, ["temperature"]}}``."""
import json
import os

# attribute -> default; grouped as the reference groups them
DEFAULTS = {
    # environment
    'target_name': None, 'codegen_type': None, 'get_op': None, 'verbose': False, 'measure_time_per_round': 32,
    'use_cost_model': True, 'out_name': 'out', 'device_id': 0, 'tuned': '',
    # sampling processes
    'parallel': True, 'parallel_num': 16,
    # population
    'pop_num': 200, 'iter_walks': 5, 'history_topk': 32,
    # cost model
    'feature_type': 'itervar', 'loss_type': 'reg',
    # genetic algorithm
    'select_num': 100, 'crossover_key_ratio': 0.2,
    # constrained GA: share of the measuring rounds, at the end, spent on one-knob neighbours of the best points
    'refine_share': 0.25,
    # constrained GA: block tiles whose best points are re-timed with long repeats when the search is over (0 = off)
    'confirm_tiles': 8,
    # ... and rounds in which the one-knob neighbours of the best confirmed point are timed the same way
    'polish_rounds': 1,
    # constrained GA: records files of earlier searches whose best rows the confirmation phase times again
    'incumbents': (),
    # simulated annealing
    'temperature': 0.6,
    # unconstrained tuners: per-variable feasible value sets from this many random feasible points (tuner.py:115-144)
    'feasible_file_path': 'feasible.json', 'feasible_samples': 1000,
    # cross-task cost model: rounds of run_with_pretrained (the reference reads it, tuner.py:36, but never defines it)
    'search_generations': 4, 'pretrained_records': (), 'pretrained_model': '',
    # what a JSON file normally supplies
    'opt_method': 'CGA', 'max_trials': 32, 'runner_number': 3, 'runner_repeat': 4, 'runner_timeout': 50,
    'build_timeout': 50, 'in_dtype': 'float16', 'out_dtype': 'float16', 'cases': (),
}

# JSON key -> attribute, for the keys every case file carries
REQUIRED_KEYS = {'out_name': 'out_name', 'method': 'opt_method', 'max_trials': 'max_trials',
                 'runner_number': 'runner_number', 'runner_repeat': 'runner_repeat', 'runner_timeout': 'runner_timeout',
                 'build_timeout': 'build_timeout', 'in_dtype': 'in_dtype', 'out_dtype': 'out_dtype', 'cases': 'cases'}
# optional keys; all but "temperature" are additions of this build
OPTIONAL_KEYS = ('temperature', 'pop_num', 'iter_walks', 'parallel_num', 'measure_time_per_round', 'select_num',
                 'history_topk', 'refine_share', 'confirm_tiles', 'polish_rounds', 'incumbents')


class Config:
    def __init__(self):
        for name, value in DEFAULTS.items():
            setattr(self, name, {} if name == 'cases' else [] if name == 'pretrained_records' else value)

    def setEnv(self, env):
        self.num_ops = env.num_ops
        self.log_dir = os.path.join(self.out_name, env.task.name)


def configFromFile(fname):
    with open(fname) as f:
        entries = json.load(f)['config']
    config = Config()
    for key, attr in REQUIRED_KEYS.items():
        setattr(config, attr, entries[key])
    for key in OPTIONAL_KEYS:
        if key in entries:
            setattr(config, key, entries[key])
    return config
