// myea_dataset_hip.hpp - the reference's epoch loops over a dataset kept in HBM.
//
// Mirrors `Dataset<T>` (Neural_Network/Dataset.cpp: Train_Epoch_Loop :593-635, Train_Batch_BP_Loop :667-700, Training
// :7574-7688, Measure_Accuracy :7690-7756, Testing :7758-7860) and `Dataset_Mini_Batch<T>` (Neural_Network/
// Dataset__Mini_Batch.cpp: Shuffle :45-66, Set__Desired_Data_Per_Batch :160-288, Increment_Mini_Batch :290-314,
// Training_Loop :381-420) on top of `Neural_Network_HIP`.  The examples are uploaded once; every batch is handed to the
// step entry points as a device pointer, and a shuffled mini-batch is gathered on the device instead of re-pointing
// an array of row pointers.  Same method names, same order of calls, same read-outs as the reference's classes.
#ifndef MYEA_DATASET_HIP_HPP
#define MYEA_DATASET_HIP_HPP

#include <cmath>
#include <cstdio>
#include <random>
#include <vector>

#include "myea_nn_hip.hpp"

namespace MyEA_HIP {

class Dataset_HIP {
public:
    Dataset_HIP() = default;
    Dataset_HIP(Dataset_HIP const &) = delete;
    Dataset_HIP &operator=(Dataset_HIP const &) = delete;
    virtual ~Dataset_HIP() { Deallocate(); }

    // rows as the reference keeps them: one pointer per example, [T * inputs] / [T * outputs] values each
    bool Allocate(size_t number_examples, size_t number_inputs, size_t number_outputs, size_t number_recurrent_depth,
                  T_ const *const *ptr_array_inputs_array, T_ const *const *ptr_array_outputs_array)
    {
        Deallocate();
        if (number_examples == 0 || number_inputs == 0 || number_outputs == 0 || number_recurrent_depth == 0) return Fail("Allocate", "empty dataset");
        p_number_examples = number_examples; p_number_inputs = number_inputs; p_number_outputs = number_outputs;
        p_number_recurrent_depth = number_recurrent_depth;
        const size_t in_row = Input_Row(), out_row = Output_Row();
        std::vector<T_> flat(number_examples * (in_row > out_row ? in_row : out_row));
        for (size_t e = 0; e < number_examples; ++e) for (size_t k = 0; k < in_row; ++k) flat[e * in_row + k] = ptr_array_inputs_array[e][k];
        if (myea_hip_device_buffer_create(number_examples * in_row, flat.data(), &dev_inputs_) != MYEA_OK) return Fail("Allocate", myea_hip_last_error());
        for (size_t e = 0; e < number_examples; ++e) for (size_t k = 0; k < out_row; ++k) flat[e * out_row + k] = ptr_array_outputs_array[e][k];
        if (myea_hip_device_buffer_create(number_examples * out_row, flat.data(), &dev_outputs_) != MYEA_OK) return Fail("Allocate", myea_hip_last_error());
        return true;
    }
    virtual bool Deallocate()
    {
        myea_hip_device_buffer_destroy(dev_inputs_); myea_hip_device_buffer_destroy(dev_outputs_);
        dev_inputs_ = dev_outputs_ = nullptr;
        return true;
    }

    // the examples one training pass works on (the whole set here, the current mini-batch in the subclass)
    virtual size_t Get__Number_Examples() const { return p_number_examples; }
    size_t Get__Number_Recurrent_Depth() const { return p_number_recurrent_depth; }
    bool Check_Topology(Neural_Network_HIP const &nn) const
    {
        myea_net_desc const &d = nn.Get__Descriptor();
        return d.layers[0].n_units == p_number_inputs && d.layers[d.n_layers - 1].n_units == p_number_outputs && d.number_recurrent_depth == p_number_recurrent_depth;
    }

    // Dataset::Training (Dataset.cpp:7574-7688): one pass over all examples, one update with (N, N)
    virtual T_ Training(Neural_Network_HIP *nn)
    {
        if (!Ready("Training", nn)) return FLT_MAX;
        nn->type_state_propagation = MYEA_STATE_TRAINING;
        Train_Epoch(nn);
        nn->Update_Parameter(Get__Number_Examples(), Get__Number_Examples());
        nn->epoch_time_step += 1.f;
        nn->Set__Loss(Neural_Network_HIP::TYPE_DATASET_TRAINING, nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_NONE));
        nn->Set__Accuracy(Neural_Network_HIP::TYPE_DATASET_TRAINING, Measure_Accuracy(Get__Number_Examples(), Get__Input_Array(), Get__Output_Array(), nn));
        nn->type_state_propagation = MYEA_STATE_INFERENCE;
        return nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_TRAINING);
    }

    // Dataset::Testing (Dataset.cpp:7758-7860): inference forward + Compute__Loss over the WHOLE set
    T_ Testing(Neural_Network_HIP *nn)
    {
        if (!Ready("Testing", nn)) return FLT_MAX;
        nn->Reset__Loss();
        const size_t n = p_number_examples, bmax = nn->batch_size;
        for (size_t first = 0; first < n; first += bmax) {
            const size_t b = first + bmax <= n ? bmax : n - first;
            nn->Forward_Pass__Device(b, dev_inputs_ + first * Input_Row());
            nn->Compute__Loss__Device(b, dev_outputs_ + first * Output_Row());
        }
        nn->number_accuracy_trial = Accuracy_Trials(n, nn);
        nn->Set__Loss(Neural_Network_HIP::TYPE_DATASET_TESTING, nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_NONE));
        nn->Set__Accuracy(Neural_Network_HIP::TYPE_DATASET_TESTING, Measure_Accuracy(n, dev_inputs_, dev_outputs_, nn));
        return nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_TESTING);
    }

    // Dataset::Measure_Accuracy (Dataset.cpp:7690-7756): counters -> percentage; the R accuracy takes a second pass
    T_ Measure_Accuracy(size_t batch_size_received, T_ const *dev_inputs, T_ const *dev_outputs, Neural_Network_HIP *nn)
    {
        if (nn->type_accuracy_function == MYEA_ACCURACY_R) {
            const size_t bmax = nn->batch_size;
            const size_t delays = p_number_recurrent_depth > 1 ? nn->number_time_delays : 0;
            nn->R_Means(batch_size_received * (p_number_recurrent_depth - delays) * nn->Get__Output_Size());
            for (size_t first = 0; first < batch_size_received; first += bmax) {
                const size_t b = first + bmax <= batch_size_received ? bmax : batch_size_received - first;
                nn->Forward_Pass__Device(b, dev_inputs + first * Input_Row());
                nn->Compute__Accuracy__R__Device(b, dev_outputs + first * Output_Row());
            }
        }
        return nn->Get__Accuracy(Neural_Network_HIP::TYPE_DATASET_NONE);
    }

protected:
    size_t p_number_examples = 0, p_number_inputs = 0, p_number_outputs = 0, p_number_recurrent_depth = 0;
    T_ *dev_inputs_ = nullptr, *dev_outputs_ = nullptr;

    size_t Input_Row() const { return p_number_inputs * p_number_recurrent_depth; }
    size_t Output_Row() const { return p_number_outputs * p_number_recurrent_depth; }
    virtual T_ const *Get__Input_Array() const { return dev_inputs_; }
    virtual T_ const *Get__Output_Array() const { return dev_outputs_; }
    static bool Fail(const char *fn, const char *what) { std::printf("%s: ERROR: %s.\n", fn, what); return false; }
    bool Ready(const char *fn, Neural_Network_HIP *nn) const
    {
        if (nn == nullptr || !nn->Use__HIP()) return Fail(fn, "the network has no device object (Set__HIP)");
        if (dev_inputs_ == nullptr) return Fail(fn, "the dataset is not allocated");
        if (!Check_Topology(*nn)) return Fail(fn, "the dataset and the network have different inputs, outputs or recurrent depth");
        return true;
    }
    size_t Accuracy_Trials(size_t examples, Neural_Network_HIP *nn) const
    {
        const size_t delays = p_number_recurrent_depth > 1 ? nn->number_time_delays : 0;
        return examples * (p_number_recurrent_depth - delays) * (nn->type_accuracy_function == MYEA_ACCURACY_CROSS_ENTROPY ? 1 : nn->Get__Output_Size());
    }

    // Train_Epoch_Loop + Train_Batch_BP_Loop (Dataset.cpp:593-700).  The dropout masks stay the caller's: draw them into
    // ptr_array_units_mask_dropout_bernoulli and push them (Copy__Dropout_Mask__Host_To_Device) before the call.
    void Train_Epoch(Neural_Network_HIP *nn)
    {
        nn->Reset__Loss();
        const bool rprop = nn->type_optimizer_function == MYEA_OPTIMIZER_IRPROP_PLUS;
        if (rprop) nn->previous_loss_rprop = nn->loss_rprop;
        const size_t n = Get__Number_Examples(), bmax = nn->batch_size;
        T_ const *x = Get__Input_Array(), *y = Get__Output_Array();
        for (size_t first = 0; first < n; first += bmax) {
            const size_t b = first + bmax <= n ? bmax : n - first;
            nn->Forward_Pass__Device(b, x + first * Input_Row());
            nn->Compute__Error__Device(b, y + first * Output_Row());
            nn->Backward_Pass(b);
            nn->Update_Derivative_Weight(b);
        }
        nn->number_accuracy_trial = Accuracy_Trials(n, nn);
        if (rprop) nn->loss_rprop = std::fabs(nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_NONE));
    }
};

class Dataset_Mini_Batch_HIP : public Dataset_HIP {
public:
    ~Dataset_Mini_Batch_HIP() override { Deallocate(); }

    // Dataset_Mini_Batch::Initialize (:93-158) + Set__Desired_Data_Per_Batch (:160-288), same double arithmetic for the
    // size of the last mini-batch
    bool Initialize(bool use_shuffle_received, size_t desired_number_examples_per_mini_batch_received, size_t number_mini_batch_maximum_received, unsigned long long seed)
    {
        if (p_number_examples == 0) return Fail("Initialize", "No data available");
        if (desired_number_examples_per_mini_batch_received == 0) return Fail("Initialize", "Desired number data per mini-batch equal zero");
        if (desired_number_examples_per_mini_batch_received > p_number_examples) return Fail("Initialize", "Desired number data per mini-batch greater than total number of data");
        double const real = static_cast<double>(p_number_examples) / static_cast<double>(desired_number_examples_per_mini_batch_received);
        size_t count = static_cast<size_t>(real);
        if (number_mini_batch_maximum_received != 0 && count > number_mini_batch_maximum_received) count = number_mini_batch_maximum_received;
        if (count <= 1) return Fail("Initialize", "Invalid number of mini-batch");
        number_mini_batch = count;
        number_examples_per_iteration = desired_number_examples_per_mini_batch_received;
        number_examples_last_iteration = number_examples = number_examples_per_iteration
                                         + static_cast<size_t>((real - static_cast<double>(count)) * static_cast<double>(number_examples_per_iteration));
        use_shuffle = use_shuffle_received;
        ptr_array_stochastic_index.resize(p_number_examples);
        for (size_t i = 0; i < p_number_examples; ++i) ptr_array_stochastic_index[i] = i;
        Generator_Random.seed(seed);
        const size_t big = number_examples_last_iteration > number_examples_per_iteration ? number_examples_last_iteration : number_examples_per_iteration;
        myea_hip_device_buffer_destroy(dev_batch_inputs_); myea_hip_device_buffer_destroy(dev_batch_outputs_);
        dev_batch_inputs_ = dev_batch_outputs_ = nullptr;
        if (myea_hip_device_buffer_create(big * Input_Row(), nullptr, &dev_batch_inputs_) != MYEA_OK ||
            myea_hip_device_buffer_create(big * Output_Row(), nullptr, &dev_batch_outputs_) != MYEA_OK) return Fail("Initialize", myea_hip_last_error());
        return true;
    }
    bool Deallocate() override
    {
        myea_hip_device_buffer_destroy(dev_batch_inputs_); myea_hip_device_buffer_destroy(dev_batch_outputs_);
        dev_batch_inputs_ = dev_batch_outputs_ = nullptr;
        return Dataset_HIP::Deallocate();
    }

    // Fisher-Yates from the top (:45-66)
    void Shuffle()
    {
        for (size_t i = p_number_examples; i-- != 0;) {
            std::uniform_int_distribution<size_t> range(0, i);
            const size_t r = range(Generator_Random);
            const unsigned long long swap = ptr_array_stochastic_index[r];
            ptr_array_stochastic_index[r] = ptr_array_stochastic_index[i];
            ptr_array_stochastic_index[i] = swap;
        }
    }
    // :290-314; the rows are copied into one contiguous device batch
    bool Increment_Mini_Batch(size_t mini_batch_iteration_received, Neural_Network_HIP *nn)
    {
        const size_t size = mini_batch_iteration_received + 1 != number_mini_batch ? number_examples_per_iteration : number_examples_last_iteration;
        const size_t first = mini_batch_iteration_received * number_examples_per_iteration, bmax = nn->batch_size;
        for (size_t off = 0; off < size; off += bmax) {   // host indices pass through a staging buffer of one maximum batch
            const size_t b = off + bmax <= size ? bmax : size - off;
            const unsigned long long *index = ptr_array_stochastic_index.data() + first + off;
            if (myea_hip_gather_examples(nn->Get__Device_Handle(), dev_batch_inputs_ + off * Input_Row(), dev_inputs_, p_number_examples, Input_Row(),
                                         reinterpret_cast<const uint64_t *>(index), 0, b) != MYEA_OK ||
                myea_hip_gather_examples(nn->Get__Device_Handle(), dev_batch_outputs_ + off * Output_Row(), dev_outputs_, p_number_examples, Output_Row(),
                                         reinterpret_cast<const uint64_t *>(index), 0, b) != MYEA_OK)
                return Fail("Increment_Mini_Batch", myea_hip_last_error());
        }
        number_examples = size;
        return true;
    }
    void Reset() { number_examples = number_examples_last_iteration; }

    size_t Get__Number_Examples() const override { return number_examples; }
    size_t Get__Number_Batch() const { return number_mini_batch; }
    size_t Get__Number_Examples_Per_Batch() const { return number_examples_per_iteration; }
    size_t Get__Number_Examples_Last_Batch() const { return number_examples_last_iteration; }
    std::vector<unsigned long long> const &Get__Stochastic_Index() const { return ptr_array_stochastic_index; }

    // Dataset_Mini_Batch::Training_Loop (:381-420)
    T_ Training(Neural_Network_HIP *nn) override
    {
        if (!Ready("Training", nn) || dev_batch_inputs_ == nullptr) return FLT_MAX;
        nn->type_state_propagation = MYEA_STATE_TRAINING;
        T_ tmp_summation_loss = 0.f, tmp_summation_accurancy = 0.f;
        if (use_shuffle) Shuffle();
        for (size_t i = 0; i != number_mini_batch; ++i) {
            if (!Increment_Mini_Batch(i, nn)) return FLT_MAX;
            Train_Epoch(nn);
            tmp_summation_loss += nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_NONE);
            tmp_summation_accurancy += Measure_Accuracy(Get__Number_Examples(), Get__Input_Array(), Get__Output_Array(), nn);
            nn->Update_Parameter(Get__Number_Examples(), Dataset_HIP::Get__Number_Examples());
        }
        Reset();
        nn->epoch_time_step += 1.f;
        nn->Set__Loss(Neural_Network_HIP::TYPE_DATASET_TRAINING, tmp_summation_loss / static_cast<T_>(number_mini_batch));
        nn->Set__Accuracy(Neural_Network_HIP::TYPE_DATASET_TRAINING, tmp_summation_accurancy / static_cast<T_>(number_mini_batch));
        nn->type_state_propagation = MYEA_STATE_INFERENCE;
        return nn->Get__Loss(Neural_Network_HIP::TYPE_DATASET_TRAINING);
    }

protected:
    T_ const *Get__Input_Array() const override { return dev_batch_inputs_; }
    T_ const *Get__Output_Array() const override { return dev_batch_outputs_; }

private:
    bool use_shuffle = true;
    size_t number_examples = 0, number_mini_batch = 0, number_examples_per_iteration = 0, number_examples_last_iteration = 0;
    std::vector<unsigned long long> ptr_array_stochastic_index;
    std::mt19937_64 Generator_Random;
    T_ *dev_batch_inputs_ = nullptr, *dev_batch_outputs_ = nullptr;
};

}  // namespace MyEA_HIP

#endif  // MYEA_DATASET_HIP_HPP
