"""Compile-only check (no GPU): a translation unit that uses the layer classes through the
reference's own names and member signatures -- LstmInputHiddenNode<float>::UpdateVectorsForwardGpu /
ForwardProp / BackPropPreprocessGpu / BackPropGpu(int), LstmHiddenHiddenNode<float>, BaseLossLayer's
BackProp1 / BackProp2 / BackPropPreprocessGpu / ComputeLossGpu (src/node_input_to_hidden.h:33-150,
src/node_hidden_to_hidden.h:30-140, src/layer_loss.h:42-103) -- compiles against host/nmt.h."""
import os
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SOURCE = r"""
#include "linmt_amd/host/nmt.h"
using namespace linmt;
typedef float precision;

// calls written the way src/deep_rnn.h:1137-1273 writes them
void target_step(NeuralMachineTranslation &m, BaseLossLayer *p_softmax_layer_,
                 InputToHiddenLayer<precision> &input_layer_target_,
                 HiddenToHiddenLayer<precision> &hidden, int i, int step) {
  LstmInputHiddenNode<precision> &n0 = input_layer_target_.v_nodes_[i];
  LstmHiddenHiddenNode<precision> &n1 = hidden.v_nodes_[i];
  p_softmax_layer_->BackPropPreprocessGpu(n1.p_device_h_t_, step);
  p_softmax_layer_->BackProp1(i);
  p_softmax_layer_->BackProp2(i);
  n1.BackPropPreprocessGpu(hidden.p_device_d_errn_to_t_ht_m1_.get(), hidden.p_device_d_errn_to_t_ct_m1_.get());
  n1.BackPropGpu(i);
  n0.BackPropPreprocessGpu(input_layer_target_.p_device_d_errn_to_t_ht_m1_.get(),
                           input_layer_target_.p_device_d_errn_to_t_ct_m1_.get());
  n0.BackPropGpu(i);
  (void)m;
}

void forward_step(InputToHiddenLayer<precision> &input_layer, HiddenToHiddenLayer<precision> &hidden,
                  BaseLossLayer *p_softmax_layer_, int *idx, int *idx01, float *h, float *c, int i) {
  input_layer.v_nodes_[i].UpdateVectorsForwardGpu(idx, idx01, h, c);
  input_layer.v_nodes_[i].ForwardProp();
  hidden.v_nodes_[i].UpdateVectorsForwardGpu(idx01, h, c);
  hidden.v_nodes_[i].ForwardProp();
  p_softmax_layer_->BackPropPreprocessGpu(hidden.v_nodes_[i].p_device_h_t_, 0);
  double loss = p_softmax_layer_->ComputeLossGpu(i);
  float *dist = p_softmax_layer_->GetDistPtr();
  (void)loss;
  (void)dist;
}
"""


def test_reference_names_and_signatures_compile():
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "uses_reference_names.cc")
        with open(src, "w") as f:
            f.write(SOURCE)
        cmd = ["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I", ROOT,
               "-I", "/opt/rocm/include", src]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
