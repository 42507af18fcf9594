"""Env: the object a driver script talks to - it owns the measurement runner, the task, the tuner and the store of
measured samples.  Interface of the reference's environment.py:10-120: ``createTask``, ``tune``, ``evalSamples``,
``get_build_kwargs`` (device limits from the runner, handed to the builder and to the schedule context)."""
import os
import shutil
import time

from .perf.perfBuffer import perfBuffer
from .runner.measure import create_measure_batch
from .runner.runner import Runner
from .schedule.sched_op import get_op_methods
from .task.task import Task
from . import tuner as tuners
from .utils import mkdir

# config "method" -> search class (CGA is the reference's own method, the others its baselines)
TUNERS = {
    'CGA': tuners.CGATuner, 'RCGA': tuners.RCGATuner, 'CRAND': tuners.CRandTuner, 'CRANDS': tuners.CRandSampler,
    'GA': tuners.GATuner, 'SRGA': tuners.SRGATuner, 'SDGA': tuners.SDGATuner, 'IDEA': tuners.IDEATuner,
    'SA': tuners.RandomWalkSATuner, 'CSA': tuners.ConstrainedRandomWalkerSATuner,
}


def create_kwargs_ctx(task, option):
    """Binds runner and builder to the task; the returned callable yields the device limits (``check_gpu``)."""
    builder, runner = option["builder"], option["runner"]
    attach_objects = runner.set_task(task)
    build_kwargs = runner.get_build_kwargs()
    builder.set_task(task, build_kwargs)

    def get():
        return build_kwargs
    get.n_parallel = builder.n_parallel
    get.attach_objects = attach_objects
    return get


class Env:
    def __init__(self, measure_option, config):
        self.config = config
        self.runner = Runner(measure_option)
        self.num_ops = len(get_op_methods(config.codegen_type))
        self.build_kwargs = None
        self.task = None
        self.tuner = None
        self.perf_buffer = None

    # ------------------------------------------------------------------ set-up
    def get_build_kwargs(self, task):
        self.build_kwargs = create_kwargs_ctx(task, self.runner.measure_option)()
        print(self.build_kwargs)

    def createTask(self, name, opfunc, args, target, target_host=None, dump_const_desc=False):
        if self.task is not None:
            raise AssertionError("an Env holds one task")
        method = self.config.opt_method
        if method not in TUNERS:
            raise ValueError('Unsupportted opt method')
        self.config.task_name = name
        task = Task(name, opfunc, args, target, target_host)
        task.knob_manager.dump_descs = dump_const_desc
        if self.build_kwargs is None:
            self.get_build_kwargs(task)
        task.build_kwargs, task.config = self.build_kwargs, self.config
        self.task = task
        self.config.setEnv(self)
        self.tuner = TUNERS[method](self.config)
        if self.config.use_cost_model:
            self.tuner.buildCostModel(task)
        self.perf_buffer = perfBuffer(self.config)
        return task

    def init_dir(self):
        if os.path.exists(self.config.log_dir):
            shutil.rmtree(self.config.log_dir)
        mkdir(self.config.log_dir)

    # ------------------------------------------------------------------ search
    def tune(self, task_name, pretrained=False):
        self.init_dir()
        started = time.time()
        self.task.make_stage_schedules()
        self.runner.measure_batch = create_measure_batch(self.task, self.runner.measure_option)
        with open(os.path.join(self.config.log_dir, 'schedule.py'), 'w') as out:
            out.write(self.task.sched_desc)
        if getattr(self.config, 'pretrained_model', ''):
            # an attention cost model fitted beforehand on the records of other tasks (tests/pretrain/train_model.py),
            # used as it is: the flow of pretrain/tune_with_pretrained.py:30-35 of the reference
            from .pretrain import AttentionCostModel
            model = AttentionCostModel().load(self.config.pretrained_model)
            print("pre-trained attention cost model: %s (%d variable names)" % (self.config.pretrained_model,
                                                                               model.vocab.size("name") - 1))
            self.tuner.setPretrainedModel(model)
            result = self.tuner.run_with_pretrained(self)
        elif pretrained or self.config.pretrained_records:
            from .model import PretrainedCostModel
            model = PretrainedCostModel(self.task, self.config)
            n = model.fit_from_records(self.config.pretrained_records, len(self.task.knob_manager.solver.vals))
            print("pre-trained cost model: %d records from %d files" % (n, len(model.files_used)))
            self.tuner.setPretrainedModel(model)
            result = self.tuner.run_with_pretrained(self)
        else:
            result = self.tuner.run(self)
        print("Heron tune time spent ", time.time() - started)
        self.runner.measure_batch = None
        return result

    def evalSamples(self, samples):
        started = time.time()
        self.runner.run(samples, self.perf_buffer)
        print("Hardware time %f" % (time.time() - started))
        return samples
