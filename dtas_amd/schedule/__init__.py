from .schedule import get_config_emiter_template, get_scheduler_template
from .tir_base import (TIRElementwiseScheduler, TIRGEMVScheduler, TIRMFMAScheduler, TIRReductionScheduler,
                       TIRSchedulerBase)
