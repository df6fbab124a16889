"""Tables of tuned operator configurations, one CSV per device.

Same file format as the reference's benchmark parameter tables
(test/bench/matmul/params/default.csv, test/bench/attention/params/default.csv):
the leading columns are lookup keys (there: granularity, sparsity), every other
column is named '<kernel>;<PARAM>' and a row flattens one `{kernel: {param: value}}`
dict as returned by tune() and accepted by build().  Reading follows
test/bench/matmul/matmul.py:157-180: `<device name>.csv` if present, else
`default.csv`; '_impl' values are strings, numeric values <= 0 mean "not set".
"""
import csv
import os
from typing import Any, Dict, Iterable, List, Optional, Tuple

ConfigDict = Dict[str, Dict[str, Any]]


def flatten_config(config: ConfigDict) -> Dict[str, Any]:
    """{'forward:C': {'_impl': 'sparta', 'BLOCK_SIZE_M_VALUE': 32}} ->
    {'forward:C;_impl': 'sparta', 'forward:C;BLOCK_SIZE_M_VALUE': 32}"""
    flat = {}
    for kernel, params in config.items():
        for name, value in params.items():
            flat[f'{kernel};{name}'] = value
    return flat


def unflatten_config(row: Dict[str, Any]) -> ConfigDict:
    """Inverse of flatten_config for one table row; key columns (no ';') are skipped."""
    config: ConfigDict = {}
    for column, value in row.items():
        if ';' not in column or value is None or value == '':
            continue
        kernel, param = column.split(';', 1)
        if param == '_impl':
            if str(value) not in ('', '0'):
                config.setdefault(kernel, {})[param] = str(value)
        else:
            number = float(value)
            if number > 0:
                config.setdefault(kernel, {})[param] = int(number)
    return config


def save_config_table(path: str, keys: List[str], rows: Iterable[Tuple[Dict[str, Any], ConfigDict]]):
    """Write `rows` = [(key values, config), ...] as one CSV.  Columns: `keys`, then the
    union of all '<kernel>;<PARAM>' columns in first-seen order; absent values stay 0."""
    rows = list(rows)
    columns: List[str] = []
    for _, config in rows:
        for column in flatten_config(config):
            if column not in columns:
                columns.append(column)
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, 'w', newline='') as f:
        writer = csv.writer(f)
        writer.writerow(list(keys) + columns)
        for key_values, config in rows:
            flat = flatten_config(config)
            writer.writerow([key_values[k] for k in keys] +
                            [flat.get(c, '' if c.endswith(';_impl') else 0) for c in columns])


def load_config_table(directory: str, device_name: Optional[str] = None) -> List[Dict[str, str]]:
    """Rows of `<directory>/<device_name>.csv` if that file exists, else of
    `<directory>/default.csv` (matmul.py:157-164 of the reference's bench)."""
    candidates = []
    if device_name:
        candidates.append(os.path.join(directory, f'{device_name}.csv'))
    candidates.append(os.path.join(directory, 'default.csv'))
    for path in candidates:
        if os.path.exists(path):
            with open(path, newline='') as f:
                return list(csv.DictReader(f))
    raise FileNotFoundError(f'no configuration table in {directory} (looked for {candidates})')


def lookup_config(table: List[Dict[str, str]], **keys) -> ConfigDict:
    """Config of the first row whose key columns equal `keys` (numbers compare as
    floats, so 0.9 matches '0.9' and 32 matches '32.0'); KeyError if there is none."""
    def same(stored: str, wanted) -> bool:
        try:
            return float(stored) == float(wanted)
        except (TypeError, ValueError):
            return str(stored) == str(wanted)

    for row in table:
        if all(k in row and same(row[k], v) for k, v in keys.items()):
            return unflatten_config(row)
    raise KeyError(f'no row with {keys}')


def packaged_table_dir(op: str) -> str:
    """Directory of the tables shipped with the package for `op` ('matmul' / 'attention')."""
    return os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'params', op)
