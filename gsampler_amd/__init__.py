"""gsampler_amd -- MI355X-native implementation of gSampler's matrix-centric
sampling hot path.  `import gsampler_amd as gs` mirrors the reference's `gs`
package for that path."""
from . import capi  # noqa: F401
