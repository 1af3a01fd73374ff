"""Mode flags the cache classes read (test infrastructure).

Follows jetstream_pt/environment.py:143-195: the derived flags
(lazy_cache_update, ragged_mha, flash_attention, generate_cache_stacked,
new_cache_stacked) are functions of ring_buffer unless `testing` is set, and
are all forced off when paging is enabled.
"""

import dataclasses

import torch


@dataclasses.dataclass
class Env:
  batch_size: int = 4
  num_layers: int = 1
  cache_len: int = 128
  bf16_enable: bool = True
  ring_buffer: bool = True
  testing: bool = False
  lazy_cache_update: bool = False
  ragged_mha: bool = False
  flash_attention: bool = False
  generate_cache_stacked: bool = False
  new_cache_stacked: bool = False
  block_size: int = 512
  paged_attention_total_num_pages: int = 0
  paged_attention_page_size: int = 64

  @property
  def cache_sequence_length(self):
    return self.cache_len

  def __post_init__(self):
    requested = (
        self.lazy_cache_update,
        self.ragged_mha,
        self.flash_attention,
        self.generate_cache_stacked,
        self.new_cache_stacked,
    )
    # environment.py:163-174
    derived = (not self.ring_buffer,) * 5
    # environment.py:176-181
    flags = requested if self.testing else derived
    self.page_attention = self.paged_attention_total_num_pages > 0
    # environment.py:183-188
    if self.page_attention:
      flags = (False,) * 5
    (
        self.lazy_cache_update,
        self.ragged_mha,
        self.flash_attention,
        self.generate_cache_stacked,
        self.new_cache_stacked,
    ) = flags
    # environment.py:190
    self.default_type = torch.bfloat16 if self.bf16_enable else torch.float32
