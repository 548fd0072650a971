from .elementwise_config_emiter import ElementwiseConfigEmiter
from .gemv_config_emiter import GEMVConfigEmiter
from .mfma_config_emiter import MFMAConfigEmiter
from .reduction_config_emiter import ReductionConfigEmiter

# the reference's name for the GEMM emitter slot
WMMAConfigEmiter = MFMAConfigEmiter
