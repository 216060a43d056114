"""aie4ml_amd — an MI355X (gfx950) executor for the quantized operators aie4ml lowers.

Public surface:
  ops            torch-tensor operator API over the HIP kernels (C ABI underneath)
  GPUModel       runtime object with the reference's compile() / predict() contract
  GraphBuilder   programmatic construction of the operator IR
  from_onnx      ONNX Q/DQ model (path / bytes) -> GPUModel, no onnx package needed
  from_hls4ml    hls4ml ModelGraph (read by attribute access, hls4ml is not imported) -> GPUModel
"""

from .aie_types import AIEDataType, QuantIntent, RoundingMode, SaturationMode
from .frontends.builder import GraphBuilder, qint
from .frontends.hls4ml_lower import from_hls4ml
from .frontends.onnx_import import from_onnx
from .model import GPUModel

__version__ = '0.1.0'
__all__ = ['AIEDataType', 'QuantIntent', 'RoundingMode', 'SaturationMode', 'GraphBuilder', 'GPUModel', 'from_hls4ml', 'from_onnx', 'qint',
           '__version__']
