#!/bin/bash
# One-process GPU test run with a per-test time limit (a hang names its test).
set -o pipefail
cd "$(dirname "$0")/.."
exec timeout -k 10 900 python -u -m pytest tests -m gpu -x -v --timeout 120 --timeout-method thread "$@"
