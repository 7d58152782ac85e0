"""bamboo_amd: one Bamboo pipeline stage (own layers forward/backward, redundant forward of the
successor's shadow layers, failover promotion) on a single MI355X, behind the reference's
``PipelineModule`` / ``initialize`` / ``PipelineEngine.train_batch`` surface.

    import bamboo_amd as deepspeed
    from bamboo_amd.pipe import PipelineModule, LayerSpec
"""
from . import hip, schedule
from .config import BambooConfig
from .layers import BottleNeck, DecoderLayer, FinalLayerNorm, MSELoss, SumLast, TransformerLayer
from .module import LayerSpec, PipelineError, PipelineModule, TiedLayerSpec
from .optim import FusedAdam
from .p2p import (AllReduceException, LocalFabric, NextStageException, PrevStageException, SeededActivationQueue,
                  StageKilled)

__version__ = "0.1.0"


def initialize(args=None, model=None, optimizer=None, model_parameters=None, training_data=None,
               lr_scheduler=None, mpu=None, dist_init_required=None, collate_fn=None, config=None,
               config_params=None, redundancy_level=0, sync_save=False, eager_recovery=False, **engine_kwargs):
    """Same signature and return tuple as the reference's ``deepspeed.initialize``
    (deepspeed/__init__.py:61-168): ``(engine, optimizer, training_dataloader, lr_scheduler)``.
    ``engine_kwargs`` carries what the one-GPU build adds: ``activation_queue`` (stand-in for the
    neighbouring stages) and ``rc_stream`` (issue redundant forwards on a second HIP stream)."""
    from .engine import PipelineEngine
    if not isinstance(model, PipelineModule):
        raise PipelineError("bamboo_amd.initialize accelerates the pipeline path only: model must be a PipelineModule")
    engine = PipelineEngine(args=args, model=model, optimizer=optimizer, model_parameters=model_parameters,
                            training_data=training_data, lr_scheduler=lr_scheduler, mpu=mpu,
                            dist_init_required=dist_init_required, collate_fn=collate_fn, config=config,
                            config_params=config_params, redundancy_level=redundancy_level, sync_save=sync_save,
                            eager_recovery=eager_recovery, **engine_kwargs)
    return engine, engine.optimizer, engine.training_data, engine.lr_scheduler


def add_config_arguments(parser):
    """``--deepspeed`` / ``--deepspeed_config`` flags of the reference scripts
    (deepspeed/__init__.py:171-240)."""
    group = parser.add_argument_group("DeepSpeed", "DeepSpeed configurations")
    group.add_argument("--deepspeed", default=False, action="store_true")
    group.add_argument("--deepspeed_config", default=None, type=str)
    return parser
