"""MI355X (gfx950) kernel backend for the eclat tensor compiler's hot path:
lowered kernel AST -> HIP C for CDNA4 -> hiprtc -> launch, behind the
reference's Backend/Device/Buffer/Kernel surface."""

__version__ = "0.1.0"
