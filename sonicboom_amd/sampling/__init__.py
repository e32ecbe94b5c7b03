from .params import SamplingParams  # noqa: F401
from .philox import philox4x32_10  # noqa: F401
from .sampler import Sampler, draw_rows, filter_candidates, gumbel_draw, penalty_items  # noqa: F401
