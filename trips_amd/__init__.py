"""MI355X-native TRIPS point-splat rasterizer: host-side mirror of the reference's operator surface
(PointRender / NeuralRenderInfo / PointRendererCache / MyAdam) over the C ABI in include/trips_splat.h."""
from . import abi, scenes  # noqa: F401

__all__ = ["abi", "scenes"]
