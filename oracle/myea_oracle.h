/* myea_oracle.h — CPU restatement of the reference's training step.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the product (the HIP library, its host adaptor) links, loads or calls this; only
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do, and only as the checker.
 *
 * The descriptor / hyper-parameter structs and enum values are the ones of include/myea_hip.h,
 * so a test feeds the same bytes to both sides.  All pointers are host pointers.
 */
#ifndef MYEA_ORACLE_H
#define MYEA_ORACLE_H

#include "../include/myea_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct myea_oracle_net myea_oracle_net;

int myea_oracle_create(const myea_net_desc *desc, myea_oracle_net **out_net);
int myea_oracle_destroy(myea_oracle_net *net);
int myea_oracle_set_hyper(myea_oracle_net *net, const myea_hyper *hyper);
int myea_oracle_get_hyper(myea_oracle_net *net, myea_hyper *hyper);
int myea_oracle_set_state_propagation(myea_oracle_net *net, uint32_t type_state_propagation);
/* number of OpenMP threads used by the batch loops (1 = the reference's __Loop variants). */
int myea_oracle_set_threads(myea_oracle_net *net, int threads);
int myea_oracle_set_unit_activations(myea_oracle_net *net, size_t layer_index, const uint32_t *types, const float *steepness, size_t count);

/* direct pointers to the flat vectors (the reference's data members are public) */
float *myea_oracle_parameters(myea_oracle_net *net);
float *myea_oracle_gradient(myea_oracle_net *net);
float *myea_oracle_optimizer_state(myea_oracle_net *net, int kind);
uint8_t *myea_oracle_masks(myea_oracle_net *net);
uint8_t *myea_oracle_zoneout_masks(myea_oracle_net *net, size_t *count);
/* Gaussian / Uout dropout draws of layer `li`, [T][Bmax][H]; NULL when the layer has no such dropout */
float *myea_oracle_dropout_noise(myea_oracle_net *net, size_t li, size_t *count);
int myea_oracle_clear_training_arrays(myea_oracle_net *net);

int myea_oracle_forward_pass(myea_oracle_net *net, size_t batch_size_received, const float *inputs);
int myea_oracle_compute_error(myea_oracle_net *net, size_t batch_size_received, const float *desired_outputs);
int myea_oracle_compute_loss(myea_oracle_net *net, size_t batch_size_received, const float *desired_outputs);
int myea_oracle_compute_accuracy_r(myea_oracle_net *net, size_t batch_size_received, const float *desired_outputs, float desired_mean, float predicted_mean);
int myea_oracle_backward_pass(myea_oracle_net *net, size_t batch_size_received);
int myea_oracle_update_derivative_weight(myea_oracle_net *net, size_t batch_size_received, size_t first_layer_index, size_t end_layer_index);
int myea_oracle_update_parameter(myea_oracle_net *net, size_t batch_size_received, size_t training_size_received);
int myea_oracle_reset_loss(myea_oracle_net *net);
int myea_oracle_get_loss(myea_oracle_net *net, myea_loss_state *out_state);

/* pointer to a layer tensor (same kinds as myea_hip_download_tensor); *count receives its length */
const float *myea_oracle_tensor(myea_oracle_net *net, size_t layer_index, int kind, size_t *count);

/* Update_Parameter__iRPROP_minus__Loop (Neural_Network__iRPROP_minus.cpp:21-67) over [0, count): the reference's own
 * Update_Parameter never dispatches it (its switch, Neural_Network.cpp:4770-4821, has no such case), so it stands alone here as
 * it does there.  previous_steps / previous_derivatives are the two vectors of that name; the gradient is zeroed. */
void myea_oracle_irprop_minus(const myea_hyper *hyper, size_t count, float *parameters, float *gradient, float *previous_steps, float *previous_derivatives);

/* scalar pieces, exported so the tests can pin them one by one */
float myea_oracle_activation(uint32_t type_activation_function, float summation);
float myea_oracle_activation_derive(uint32_t type_activation_function, float summation, float steepness, float value);

#ifdef __cplusplus
}
#endif
#endif
