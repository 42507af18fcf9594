"""Tuning configuration: defaults and JSON schema of the reference (config.py:4-54)."""
import json
import os


class Config:
    def __init__(self):
        # Environment configs
        self.target_name = None
        self.codegen_type = None
        self.get_op = None
        self.verbose = False
        self.measure_time_per_round = 32
        self.use_cost_model = True
        self.out_name = 'out'
        self.device_id = 0
        self.tuned = ''

        self.parallel = True
        self.parallel_num = 16

        # Common
        self.pop_num = 200
        self.iter_walks = 5
        self.history_topk = 32

        # cost model configs
        self.feature_type = 'itervar'
        self.loss_type = 'reg'

        # Genetic algorithm params
        self.select_num = 100
        self.crossover_key_ratio = 0.2

        # Simulated annealing params
        self.temperature = 0.6

        self.feasible_file_path = 'feasible.json'
        self.search_generations = 4           # rounds of run_with_pretrained (tuner.py:36; the reference leaves it undefined)
        self.pretrained_records = []          # records.txt files of earlier tasks for the cross-task cost model
        self.feasible_samples = 1000          # random feasible points behind the per-variable value sets (tuner.py:115)

        # defaults for configs created in code rather than from a file
        self.opt_method = 'CGA'
        self.max_trials = 32
        self.runner_number = 3
        self.runner_repeat = 4
        self.runner_timeout = 50
        self.build_timeout = 50
        self.in_dtype = 'float16'
        self.out_dtype = 'float16'
        self.cases = {}

    def setEnv(self, env):
        self.num_ops = env.num_ops
        self.log_dir = os.path.join(self.out_name, env.task.name)


def configFromFile(fname):
    with open(fname, "r") as f:
        data = json.load(f)
    config = Config()
    c = data['config']
    config.out_name = c['out_name']
    config.opt_method = c['method']
    config.max_trials = c['max_trials']
    config.runner_number = c['runner_number']
    config.runner_repeat = c['runner_repeat']
    config.runner_timeout = c['runner_timeout']
    config.build_timeout = c['build_timeout']
    config.in_dtype = c['in_dtype']
    config.out_dtype = c['out_dtype']
    config.cases = c['cases']
    if "temperature" in c.keys():
        config.temperature = c["temperature"]
    # optional overrides of the search defaults (not in the reference's schema)
    for key in ("pop_num", "iter_walks", "parallel_num", "measure_time_per_round", "select_num", "history_topk"):
        if key in c:
            setattr(config, key, c[key])
    return config
