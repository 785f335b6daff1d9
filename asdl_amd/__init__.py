"""MI355X-native K-FAC / Shampoo curvature path behind the GradientMaker API of kazukiosawa/asdl.

The public names below match the reference package (``asdl``) for this path; the arithmetic runs in
hand-written gfx950 HIP kernels (asdl_amd/csrc) loaded through a C ABI (include/asdl_amd.h).
"""
from .matrices import *
from .grad_maker import GradientMaker, DummyObject, LOSS_CROSS_ENTROPY, LOSS_MSE
from .utils import cholesky_inv, im2col_2d, skip_param_grad, has_reduction, original_requires_grad
from .symmatrix import SymMatrix, Kron, UnitWise, matrix_to_tril, tril_to_matrix, get_n_cols_by_tril
from .operations import (Operation, Linear, Conv2d, BatchNorm, LayerNorm, OperationContext, get_op_class, OP_COV_KRON,
                         OP_COV_KRON_INV, OP_COV_SWIFT_KRON, OP_COV_SWIFT_KRON_INV, OP_COV_UNIT_WISE, OP_COV_UNIT_WISE_INV,
                         OP_SAVE_INPUTS, OP_SAVE_OUTPUTS, OP_SAVE_OUTGRADS)
from .core import extend, no_centered_cov, module_wise_assignments, modules_to_assign
from .fisher import FisherConfig, get_fisher_maker, FisherMaker
from .prec_grad_maker import (PreconditionedGradientMaker, PreconditioningConfig, get_update_schedule,
                              INTERVAL_CONSTANT, INTERVAL_STEP, INTERVAL_LINEAR, INTERVAL_TYPES)
from .natural_gradient import NaturalGradientMaker, KfacGradientMaker
from .shampoo import ShampooGradientMaker, Preconditioner, BlockPartitioner, compute_power
from . import kernels
