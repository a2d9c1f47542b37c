import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, 'ocnn-pytorch_amd')):
  if p not in sys.path:
    sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, 'tests', 'golden')
REF_DATA = os.path.join(GOLDEN, 'ref_data')


def pytest_configure(config):
  config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


@pytest.fixture(scope='session')
def ref_data():
  return REF_DATA


def random_cases(default):
  """The case numbers (= seeds) of a random parity test: `default` of them from 0 on, or
  OCNN_TEST_CASES of them from OCNN_TEST_FIRST on (a sweep continues where another one ended)."""
  first = int(os.environ.get('OCNN_TEST_FIRST', '0'))
  return range(first, first + int(os.environ.get('OCNN_TEST_CASES', str(default))))
