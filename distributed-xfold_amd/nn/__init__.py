"""Drop-in modules for the reference's hot-path `nn` classes
(src/distributed_xfold/nn/*): same constructor keywords, parameter names and
`forward` signatures; `forward` runs the HIP kernels."""

from .base import HipModule, check_mode, enable_hip, in_check_mode
from .triangle_multiplication import TriangleMultiplication
from .attention import GridSelfAttention
from .primitives import Transition
from .diffusion_transformer import (AdaptiveLayerNorm, AdaLNZero, DiffusionTransition, SelfAttention,
                                    DiffusionTransformer, CrossAttention, DiffusionCrossAttTransformer)
from .pairformer import PairformerBlock, PairformerStack, pairformer_loop
from .evoformer import OuterProductMean, MSAAttention, EvoformerBlock
from .trunk import Evoformer
from . import atom_layout
from .atom_cross_attention import AtomCrossAttEncoder, AtomCrossAttDecoder, AtomCrossAttEncoderOutput
from .diffusion_head import DiffusionHead, DiffusionSampler, FourierEmbeddings

# names used by the reference for the same modules
XSMMTriangleMultiplication = TriangleMultiplication
DistributeTriangleMultiplication = TriangleMultiplication
DistributeGridSelfAttention = GridSelfAttention
DistributeTransition = Transition
DistributeAdaLNZero = AdaLNZero
DistributeDiffusionTransition = DiffusionTransition
DistributeSelfAttention = SelfAttention
DistributeDiffusionTransformer = DiffusionTransformer
DistrubuteCrossAttention = CrossAttention
DistributeDiffusionCrossAttTransformer = DiffusionCrossAttTransformer
DistributePairformerBlock = PairformerBlock
DistributeOuterProductMean = OuterProductMean
DistributeMSAAttention = MSAAttention
DistributeEvoformerBlock = EvoformerBlock
DistributeEvoformer = Evoformer
DistributeAtomCrossAttEncoder = AtomCrossAttEncoder
DistributeAtomCrossAttDecoder = AtomCrossAttDecoder
DistributeDiffusionHead = DiffusionHead
DistrubuteFourierEmbeddings = FourierEmbeddings

__all__ = [
    "HipModule", "enable_hip", "check_mode", "in_check_mode", "TriangleMultiplication", "GridSelfAttention", "Transition",
    "AdaptiveLayerNorm", "AdaLNZero", "DiffusionTransition", "SelfAttention", "DiffusionTransformer",
    "CrossAttention", "DiffusionCrossAttTransformer", "PairformerBlock", "PairformerStack", "pairformer_loop",
    "OuterProductMean", "MSAAttention", "EvoformerBlock", "Evoformer",
    "atom_layout", "AtomCrossAttEncoder", "AtomCrossAttDecoder", "AtomCrossAttEncoderOutput", "DiffusionHead",
    "DiffusionSampler", "FourierEmbeddings",
]
