"""Names of the curvature types and shapes (same strings as asdl/matrices.py:10-21)."""
HESSIAN = 'hessian'
FISHER_EXACT = 'fisher_exact'
FISHER_MC = 'fisher_mc'
FISHER_EMP = 'fisher_emp'

SHAPE_FULL = 'full'
SHAPE_LAYER_WISE = 'layer_wise'
SHAPE_KRON = 'kron'
SHAPE_SWIFT_KRON = 'swift_kron'
SHAPE_KFE = 'kfe'
SHAPE_UNIT_WISE = 'unit_wise'
SHAPE_DIAG = 'diag'

__all__ = ['HESSIAN', 'FISHER_EXACT', 'FISHER_MC', 'FISHER_EMP', 'SHAPE_FULL', 'SHAPE_LAYER_WISE', 'SHAPE_KRON',
           'SHAPE_SWIFT_KRON', 'SHAPE_KFE', 'SHAPE_UNIT_WISE', 'SHAPE_DIAG']
