"""psi-dec_amd: the MI355X (gfx950) paged KV-cache attention path behind the reference's GQA
component interface.  The directory name carries a hyphen, so load it with
`importlib.import_module("psi-dec_amd")`.
"""
from ._lib import (  # noqa: F401
    BF16,
    F16,
    F32,
    LIB_PATH,
    PROTOTYPES,
    SENTINEL,
    PsiHipError,
    load,
)
from .gqa import *  # noqa: F401,F403
from .gqa import (  # noqa: F401
    Device,
    Dtype,
    GQAActivationGateKernel,
    GQAKVPageWrite,
    GQAKVPageWriteBuffers,
    GQAKVPageWriteConfig,
    GQAKVPageWriteShape,
    GQAMetadataBuffers,
    GQAPageTableLayout,
    GQAQGKVSplitKernel,
    GQAReplayBucketPolicy,
    GQAReplayShape,
    GQARequestPageTable,
    GQASplitKV,
    GQASplitKVConfig,
    GQASplitKVSingleQConfig,
    GQASplitKVSingleQKernels,
    GQASplitKVSingleQScratch,
    GQASplitKVSingleQShape,
    GQASplitKVTiledQConfig,
    GQASplitKVTiledQKernels,
    GQASplitKVTiledQScratch,
    GQASplitKVTiledQShape,
    GQASplitKVVariant,
    OutputGate,
    ReplayBucketPolicy,
    RMSNormRopeConfig,
    RMSNormRopeKernel,
    RopeScaling,
    balanced_workers,
    select_split_kv_variant,
)
