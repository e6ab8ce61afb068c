#!/bin/bash
# Same entry-point name as the reference's cpp/build_all_bindings.sh; builds the one
# C-ABI library that all binding modules in this directory wrap.
set -e
cd "$(dirname "$0")"
python3 build.py "$@"
