"""MI355X-native dynamic-k MoE-FFN forward: the reference's MoE-layer interface over hand-written gfx950 kernels."""
from .experts import MOE_IMPL_MAP, ExpertsLayer, HipExecuteAllExperts, HipKernelExperts, init_
from .hip_abi import D2DMoEError
from .layer import ACTIVATION_NAME_MAP, MoELayer, MoeficationMoE, MoeficationRouter, add_routers
from .checkpoint import load_model_state, prepack, read_model_state, strip_wrapper_prefixes

__all__ = ['MOE_IMPL_MAP', 'ExpertsLayer', 'HipExecuteAllExperts', 'HipKernelExperts', 'init_', 'D2DMoEError',
           'ACTIVATION_NAME_MAP', 'MoELayer', 'MoeficationMoE', 'MoeficationRouter', 'add_routers',
           'read_model_state', 'load_model_state', 'strip_wrapper_prefixes', 'prepack']
