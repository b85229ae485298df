#!/bin/bash
# Builds libparamsp_hip.so (hipcc, gfx950) and the three PyTorch extension modules ParamSpMM, ParamSDDMM and
# ParamSpCONV into paramspmm_ae_amd/lib/.  Same role as the reference's script/build_param.sh.
set -e
cd "$(dirname "$0")/.."
python -m paramspmm_ae_amd.build "$@"
echo "add $(pwd)/paramspmm_ae_amd/lib to PYTHONPATH to import ParamSpMM / ParamSDDMM / ParamSpCONV"
