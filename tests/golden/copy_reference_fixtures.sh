#!/bin/sh
# Copies the data files the reference's unit tests read into tests/golden/reference_fixtures/.
# Run in the build container only (the reference tree does not exist on the GPU box).
set -e
here=$(cd "$(dirname "$0")" && pwd)
ref=${1:-/root/reference}
mkdir -p "$here/reference_fixtures/input" "$here/reference_fixtures/output"
cp "$ref"/tests/input/*.txt "$here/reference_fixtures/input/"
cp "$ref"/tests/output/*.txt "$ref"/tests/output/dropout_backward "$here/reference_fixtures/output/"
