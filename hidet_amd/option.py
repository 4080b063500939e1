"""The three option knobs the quantized-matmul path reads, with the reference's names and defaults
(python/hidet/option.py:163, 329, 366-369, 1058-1088)."""
from typing import Union

_OPTIONS = {'parallel_k': 'disabled', 'search_space': 0, 'hip.arch': 'gfx950'}


def parallel_k(strategy: Union[str, int] = 'default'):
    """'default' | 'disabled' | 'search' | an integer number of K parts (python/hidet/option.py:1058-1088)."""
    if not (isinstance(strategy, int) or strategy in ('default', 'disabled', 'search')):
        raise ValueError('invalid parallel_k: {}'.format(strategy))
    _OPTIONS['parallel_k'] = strategy


def get_parallel_k() -> Union[str, int]:
    return _OPTIONS['parallel_k']


def search_space(space: int):
    if space not in (0, 1, 2):
        raise ValueError('search space must be 0, 1 or 2')
    _OPTIONS['search_space'] = space


def get_search_space() -> int:
    return _OPTIONS['search_space']


class hip:  # namespace, as hidet.option.hip
    @staticmethod
    def arch(arch: str = 'auto'):
        if arch not in ('auto', 'gfx950'):
            raise ValueError('this library is built for gfx950 only, got {}'.format(arch))
        _OPTIONS['hip.arch'] = 'gfx950'

    @staticmethod
    def get_arch() -> str:
        return _OPTIONS['hip.arch']
