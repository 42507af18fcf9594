"""Env: owns the runner, the task, the tuner and the perf buffer (environment.py:10-120 of the reference)."""
import os
import shutil
import time

from .perf.perfBuffer import perfBuffer
from .runner.measure import create_measure_batch
from .runner.runner import Runner
from .schedule.sched_op import get_op_methods
from .task.task import Task
from .tuner import (CGATuner, ConstrainedRandomWalkerSATuner, CRandSampler, CRandTuner, GATuner, IDEATuner, RCGATuner,
                    RandomWalkSATuner, SDGATuner, SRGATuner)
from .utils import mkdir


class Env:
    def __init__(self, measure_option, config):
        self.config = config
        self.runner = Runner(measure_option)
        op_methods = get_op_methods(config.codegen_type)
        self.num_ops = len(op_methods.keys())
        self.build_kwargs = None
        self.task = None

    def init_dir(self):
        if os.path.exists(self.config.log_dir):
            shutil.rmtree(self.config.log_dir)
        mkdir(self.config.log_dir)

    def get_build_kwargs(self, task):
        get = create_kwargs_ctx(task, self.runner.measure_option)
        self.build_kwargs = get()
        print(self.build_kwargs)

    def tune(self, task_name, pretrained=False):
        self.init_dir()
        start = time.time()
        self.task.make_stage_schedules()
        self.runner.measure_batch = create_measure_batch(self.task, self.runner.measure_option)
        self.dump_schedule()
        if pretrained or self.config.pretrained_records:
            from .model import PretrainedCostModel
            model = PretrainedCostModel(self.task, self.config)
            n = model.fit_from_records(self.config.pretrained_records, len(self.task.knob_manager.solver.vals))
            print("pre-trained cost model: %d records from %d files" % (n, len(model.files_used)))
            self.tuner.setPretrainedModel(model)
            res = self.tuner.run_with_pretrained(self)
        else:
            res = self.tuner.run(self)
        print("Heron tune time spent ", time.time() - start)
        del self.runner.measure_batch
        return res

    def dump_schedule(self):
        with open(os.path.join(self.config.log_dir, 'schedule.py'), 'w') as f:
            f.write(self.task.sched_desc)

    def createTask(self, name, opfunc, args, target, target_host=None, dump_const_desc=False):
        assert self.task is None
        self.config.task_name = name
        task = Task(name, opfunc, args, target, target_host)
        task.knob_manager.dump_descs = dump_const_desc
        if self.build_kwargs is None:
            self.get_build_kwargs(task)
        task.build_kwargs = self.build_kwargs
        task.config = self.config
        self.task = task

        self.config.setEnv(self)
        method = self.config.opt_method
        tuners = {'CRAND': CRandTuner, 'CRANDS': CRandSampler, 'CGA': CGATuner, 'RCGA': RCGATuner, 'GA': GATuner,
                  'SRGA': SRGATuner, 'SDGA': SDGATuner, 'IDEA': IDEATuner, 'SA': RandomWalkSATuner,
                  'CSA': ConstrainedRandomWalkerSATuner}
        if method not in tuners:
            raise ValueError('Unsupportted opt method')
        self.tuner = tuners[method](self.config)
        if self.config.use_cost_model:
            self.tuner.buildCostModel(self.task)
        self.perf_buffer = perfBuffer(self.config)
        return task

    def evalSamples(self, samples):
        start = time.time()
        self.runner.run(samples, self.perf_buffer)
        print("Hardware time %f" % (time.time() - start))
        return samples


def create_kwargs_ctx(task, option):
    builder = option["builder"]
    runner = option["runner"]
    attach_objects = runner.set_task(task)
    build_kwargs = runner.get_build_kwargs()
    builder.set_task(task, build_kwargs)

    def get():
        return build_kwargs
    get.n_parallel = builder.n_parallel
    get.attach_objects = attach_objects
    return get
