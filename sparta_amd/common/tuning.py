"""Search-space leaf used by every tunable kernel parameter.

Mirrors sparta/common/tuning.py:10-75 (TunableItemCfg).  The NNI wrapper of the
reference (tuning.py:78-119) is not part of the operator path and is not
provided.
"""
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Union

from sparta_amd.common.utils import check_type


@dataclass
class TunableItemCfg:
    """A `choice` over a flat list of values, or (nested) over named sub-spaces
    whose entries are themselves TunableItemCfg."""
    _type: str
    _value: Union[Dict, List]
    _is_nested: Optional[bool] = False

    def __post_init__(self):
        assert self._type in ('choice',), f'unsupported space type {self._type}'
        if not self._is_nested:
            check_type(self._value, list)
            return
        check_type(self._value, dict)
        for sub_space in self._value.values():
            check_type(sub_space, dict)
            for leaf in sub_space.values():
                check_type(leaf, TunableItemCfg)

    def includes(self, value: Any) -> bool:
        return (not self._is_nested) and value in self._value

    def to_nni_search_space(self):
        """Plain-dict form: {'_type': ..., '_value': ...}; nested spaces become a
        list of {'_name': sub_space, **params} dicts."""
        if not self._is_nested:
            return {'_type': self._type, '_value': self._value}
        flat = [
            {'_name': name, **{k: v.to_nni_search_space() for k, v in params.items()}}
            for name, params in self._value.items()
        ]
        return {'_type': self._type, '_value': flat}
