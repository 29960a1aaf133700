"""The engine's own configuration (no GPU): defaults after the reference's rules, validation, and what
the scheduler and the step function make of ``max_model_len``."""
import pytest

from torchlet_amd.cache.manager import CacheManager
from torchlet_amd.engine.config import EngineConfig
from torchlet_amd.engine.request import Request
from torchlet_amd.engine.scheduler import Scheduler
from torchlet_amd.parts.base import PagedNeed


def test_defaults_follow_the_reference_and_memory_caps_them():
    """/root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:40-47: pages per request =
    ceil(max positions / page), pool = slots * that + 1 unless given."""
    c = EngineConfig(max_slots=4, page_size=16)
    assert c.resolve(32768, 1000, None).num_pages == 4 * 2048 + 1
    assert c.resolve(100, 1000, None).num_pages == 4 * 7 + 1
    assert EngineConfig(max_slots=64, max_model_len=4096).resolve(32768, 1000, None).num_pages == 64 * 256 + 1
    assert EngineConfig(max_slots=64, max_model_len=10 ** 6).model_len(32768) == 32768
    assert c.resolve(32768, 1 << 20, 1 << 30).num_pages == int((1 << 30) * 0.8) >> 20       # 0.8 of the free memory
    assert EngineConfig(num_pages=77).resolve(32768, 1, 1).num_pages == 77                  # given: kept
    assert c.resolve(32768, 1 << 30, 1 << 20).num_pages == 2                                # never below one usable page


@pytest.mark.parametrize("bad", [dict(page_size=0), dict(max_slots=0), dict(max_tokens_per_step=-1), dict(num_pages=1),
                                 dict(max_model_len=0), dict(memory_fraction=0.0), dict(memory_fraction=1.5),
                                 dict(dtype="bfloat16", kv_dtype="float32"), dict(page_size=True)])
def test_invalid_configurations_are_refused(bad):
    with pytest.raises(ValueError):
        EngineConfig(**bad)
    assert EngineConfig(dtype="bf16", kv_dtype="bfloat16").kv_dtype == "bfloat16"


def test_max_model_len_bounds_requests_at_the_scheduler():
    need = PagedNeed(num_heads=1, head_dim=16)
    cache = CacheManager([(need, None, None)], page_size=16, num_pages=100, max_requests=2)
    s = Scheduler(cache, max_tokens_per_step=64, max_positions=EngineConfig(max_model_len=50).model_len(4096))
    s.add_request(Request(prompt_tokens=[1] * 40, max_new_tokens=11))        # 40 + 11 - 1 = 50 positions
    with pytest.raises(ValueError, match="50"):
        s.add_request(Request(prompt_tokens=[1] * 40, max_new_tokens=12))
