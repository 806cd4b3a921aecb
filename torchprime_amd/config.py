"""A minimal stand-in for the OmegaConf ``DictConfig`` objects the reference passes around.

The hot-path modules read their config with attribute access *and* ``"key" in config``
(torchprime/torch_xla_models/attention.py:46-49, 75); ``Config`` supports both, plus ``get`` and item
access, so a plain ``dict`` of hyper-parameters can be used where the reference builds a DictConfig.
Real DictConfig objects work too; nothing here imports omegaconf.
"""

from __future__ import annotations

from collections.abc import Mapping


class Config(Mapping):
  def __init__(self, *args, **kwargs):
    for k, v in dict(*args, **kwargs).items():
      setattr(self, k, Config(v) if isinstance(v, dict) else v)

  def __getitem__(self, key):
    try:
      return self.__dict__[key]
    except KeyError:
      raise KeyError(key) from None

  def __iter__(self):
    return iter(self.__dict__)

  def __len__(self):
    return len(self.__dict__)

  def __contains__(self, key):
    return key in self.__dict__

  def __repr__(self):
    return f"Config({self.__dict__!r})"


def has_key(config, key: str) -> bool:
  """``key in config`` for DictConfig / Mapping / plain namespaces alike."""
  try:
    return key in config
  except TypeError:
    return hasattr(config, key)
