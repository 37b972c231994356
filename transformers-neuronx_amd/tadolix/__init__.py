"""The Tadolix design: several copies of the residual stream that every sublayer reads a weighted sum of and
writes back into through a small mixing matrix (hyper-connections), sines and cosines of the position added to the
scaled token rows, a short causal convolution over time on what a mixer reads, and layers whose mixer is either a
pair side by side (softmax attention inside chunks of the sequence, with unit-norm queries and keys, capped
scores, a learned bias by distance and an output gate, beside a minimal gated recurrence) or Griffin's recurrent
block with a real-gated linear recurrence; a gated feed-forward where a layer has one; and a stretch of layers
that is run several times over with the same weights. Importing the package registers the architecture."""
from .config import TadolixConfig  # noqa: F401
from .spec import ARCHITECTURE, tadolix_spec  # noqa: F401
