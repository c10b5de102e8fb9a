from .matmul.sparse_low_precision import *
from .matmul.bmm import *
from .matmul.sbmm import *
from .matmul.lora import *
from .matmul.ldmm import ldmm, baseline_ldmm
from .utils.sparsity import mask_creator
from .utils.generator import *
