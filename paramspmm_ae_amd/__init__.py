"""MI355X-native ParamSpMM / ParamSDDMM.

Layout:
  csrc/            HIP kernels + the C ABI (libparamsp_hip.so) and the PyTorch extension glue
  lib/             build output: libparamsp_hip.so, ParamSpMM.so, ParamSDDMM.so, ParamSpCONV.so
  graph_input.py   PCSR format builder            (surface of the reference's graph_input.py)
  PCSR.py          operator facade pcsr_spmm      (surface of the reference's PCSR.py)
  decider.py       SpMMDecider                    (surface of the reference's decider.py)
  gnn_conv.py      GCN / GIN / AGNN layers        (surface of the reference's gnn_conv.py)
  GNN.py           training driver                (surface of the reference's GNN.py)
  verification.py  torch.sparse.mm comparison     (surface of the reference's verification.py)
  synth.py         seeded synthetic graph generators

The extension modules keep the reference's top-level names: importing this package puts lib/ on sys.path
so that `import ParamSpMM`, `import ParamSDDMM`, `import ParamSpCONV` resolve to this build.
"""
import os
import sys

LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
if LIB_DIR not in sys.path:
    sys.path.insert(0, LIB_DIR)
