"""The slice of the engine environment the KV-cache path reads.

Mirrors the fields of JetEngineEnvironment that cache_manager.py, layers.py
and attention_kernel.py consult (reference: jetstream_pt/environment.py
:143-195): batch_size, num_layers, the mode flags derived from `ring_buffer`
(independently settable only under `testing`), paging parameters and the
activation dtype.  Mesh and sharding members exist so reference call sites
keep working; on one GPU they do nothing.
"""

import dataclasses

import torch


@dataclasses.dataclass
class JetEngineEnvironmentData:
  batch_size: int = 32
  cache_sequence_length: int = 2048
  num_layers: int = 0
  bf16_enable: bool = True
  ring_buffer: bool = True
  ragged_mha: bool = False
  flash_attention: bool = False
  generate_cache_stacked: bool = False
  new_cache_stacked: bool = False
  lazy_cache_update: bool = False
  block_size: int = 512
  paged_attention_total_num_pages: int = 0
  paged_attention_page_size: int = 64
  shard_on_batch: bool = False
  testing: bool = False
  testing_seed: int = 0
  cache_shape: tuple = ()


class JetEngineEnvironment:

  def __init__(self, data: JetEngineEnvironmentData = None, **overrides):
    data = dataclasses.replace(data or JetEngineEnvironmentData(), **overrides)
    self._data = data
    self.batch_size = data.batch_size
    self.cache_len = data.cache_sequence_length
    self.block_size = data.block_size
    self.num_layers = data.num_layers
    self.testing = data.testing
    self.testing_seed = data.testing_seed
    self.ring_buffer = data.ring_buffer
    self.page_attention = data.paged_attention_total_num_pages > 0
    derived = not data.ring_buffer  # environment.py:163-174
    flags = dict(lazy_cache_update=derived, ragged_mha=derived, flash_attention=derived,
                 generate_cache_stacked=derived, new_cache_stacked=derived)
    if data.testing:  # environment.py:176-181
      flags = {k: getattr(data, k) for k in flags}
    if self.page_attention:  # environment.py:183-188
      flags = {k: False for k in flags}
    for k, v in flags.items():
      setattr(self, k, v)
    self.default_type = torch.bfloat16 if data.bf16_enable else torch.float32
    self.cache_shape = ((self.num_layers, *data.cache_shape)
                        if self.generate_cache_stacked else tuple(data.cache_shape))
    self.mesh = None
    self.cache_sharding_axis = None
    self.cache_sharding = None

  def __getattr__(self, name):
    return getattr(self.__dict__["_data"], name)

  def apply_sharding(self, tensor, *, axis=None):
    return None

  def partition_by_axis(self, axis=None):
    return None

  def sharding_by_axis(self, axis):
    return None
