// myea_lstm.hip — LSTM-with-peephole layers (placeholder until the BPTT kernels land).
#include "myea_kernels.h"
#include "myea_net.h"

namespace myea {

int Net::lstm_create_layer(size_t li) { set_last_error("layer %zu: LSTM layers are not built yet", li); return MYEA_E_UNSUPPORTED; }
void Net::lstm_destroy_layer(DevLayer &) {}
int Net::lstm_parameters_changed() { return MYEA_OK; }
int Net::lstm_forward_layer(size_t li, size_t) { set_last_error("layer %zu: LSTM forward not built", li); return MYEA_E_UNSUPPORTED; }
int Net::lstm_backward_into_layer(size_t li, size_t) { set_last_error("layer %zu: LSTM backward not built", li); return MYEA_E_UNSUPPORTED; }
int Net::lstm_backward_layer(size_t li, size_t) { set_last_error("layer %zu: LSTM backward not built", li); return MYEA_E_UNSUPPORTED; }
int Net::lstm_update_derivative_weight(size_t li, size_t) { set_last_error("layer %zu: LSTM dW not built", li); return MYEA_E_UNSUPPORTED; }
const float *Net::lstm_tensor(size_t, int, size_t *count) { if (count) *count = 0; return nullptr; }

}  // namespace myea
