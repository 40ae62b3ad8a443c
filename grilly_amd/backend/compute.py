"""`Compute()`: the facade object of the reference (backend/compute.py:23-54) for the
transformer-forward path: `.fnn`, `.attention`, the convenience delegates of
backend/compute.py:153-195, `cleanup()` and `set_architecture()`."""
from .core import HipCore
from .fnn import HipFNN
from .attention import HipAttention
from .embedding import HipLearning, HipPooling


class HipCompute:
    def __init__(self, device=0, architecture=None):
        self.core = HipCore(device)
        self.architecture = architecture
        self.fnn = HipFNN(self.core)
        self.attention = HipAttention(self.core, architecture)
        # the encoder's first and last step (reference compute.py:44, :47 bind whole namespaces; only these two methods are on the path)
        self.learning = HipLearning(self.core)
        self.pooling = HipPooling(self.core)
        # always present here; the reference only binds it after set_architecture (compute.py:99)
        self.flash_attention2 = self.attention.flash_attention2
        self.flash_attention2_rope = self.attention.flash_attention2_rope

    def set_architecture(self, architecture):
        """Accepted for compatibility (reference compute.py:70-79 only selects attention-output
        shader variants, which this path does not use)."""
        self.architecture = architecture
        self.attention.architecture = architecture

    def cleanup(self):
        self.core.cleanup()

    def device_info(self):
        return self.core.device_info()

    # delegates (reference backend/compute.py:153-195)
    def linear(self, *a, **k): return self.fnn.linear(*a, **k)
    def gemm(self, *a, **k): return self.fnn.gemm(*a, **k)
    def layernorm(self, *a, **k): return self.fnn.layernorm(*a, **k)
    def residual(self, *a, **k): return self.fnn.residual(*a, **k)
    def activation_gelu(self, *a, **k): return self.fnn.activation_gelu(*a, **k)
    def activation_silu(self, *a, **k): return self.fnn.activation_silu(*a, **k)
    def activation_relu(self, *a, **k): return self.fnn.activation_relu(*a, **k)
    def activation_swiglu(self, *a, **k): return self.fnn.activation_swiglu(*a, **k)
    def activation_gcu(self, *a, **k): return self.fnn.activation_gcu(*a, **k)
    def activation_roswish(self, *a, **k): return self.fnn.activation_roswish(*a, **k)
    def activation_softmax(self, *a, **k): return self.fnn.activation_softmax(*a, **k)
    def fused_linear_gelu(self, *a, **k): return self.fnn.fused_linear_gelu(*a, **k)
    def fused_linear_silu(self, *a, **k): return self.fnn.fused_linear_silu(*a, **k)
    def fused_swiglu(self, *a, **k): return self.fnn.fused_swiglu(*a, **k)
    def fused_linear_relu(self, *a, **k): return self.fnn.fused_linear_relu(*a, **k)
    def fused_reglu(self, *a, **k): return self.fnn.fused_reglu(*a, **k)
    def fused_geglu(self, *a, **k): return self.fnn.fused_geglu(*a, **k)
    def apply_rope(self, *a, **k): return self.attention.apply_rope(*a, **k)
    def embedding_lookup(self, *a, **k): return self.learning.embedding_lookup(*a, **k)     # reference compute.py:324-326

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.cleanup()


Compute = HipCompute
