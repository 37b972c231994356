"""The Zotunex design: pre-norm layers whose norms carry one number each, the mixer either softmax attention whose
values are its keys as projected (grouped heads, a norm a head on queries and keys, partly turned heads with
stretched positions, a number a head on the scores, a gate a head on the result) or latent attention with a sink in
its softmax, the feed-forward dense with a squared relu or a mixture of clamped gated experts chosen by corrected
sigmoid scores beside a shared one. Importing the package registers the architecture."""
from .config import ZotunexConfig  # noqa: F401
from .spec import ARCHITECTURE, zotunex_spec  # noqa: F401
