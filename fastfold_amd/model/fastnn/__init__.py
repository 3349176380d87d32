"""Drop-in surface of the reference's ``fastfold.model.fastnn`` for the Evoformer path and the two
stacks that feed it (extra-MSA, template pair) (fastnn/__init__.py:1-13)."""
from .msa import MSACore, ExtraMSACore, ExtraMSABlock, ExtraMSAStack
from .ops import OutProductMean, set_chunk_size, get_chunk_size
from .triangle import PairCore
from .evoformer import Evoformer, EvoformerStack
from .template import TemplatePairBlock, TemplatePairStack, TemplatePointwiseAttention

__all__ = ['MSACore', 'OutProductMean', 'PairCore', 'set_chunk_size', 'get_chunk_size', 'Evoformer', 'EvoformerStack',
           'ExtraMSACore', 'ExtraMSABlock', 'ExtraMSAStack', 'TemplatePairBlock', 'TemplatePairStack', 'TemplatePointwiseAttention']
