// thundergbm-predict: load "tgbm.model", load LIBSVM data, predict and log the metric (the
// reference's src/thundergbm/thundergbm_predict.cpp).
#include "host.h"

using namespace tgbm;

int main(int argc, char **argv) {
    GBMParam param;
    Parser::parse_param(param, argc, argv);
    g_verbose = param.verbose;
    DataSet dataset;
    std::vector<std::vector<Tree>> model;
    Parser::load_model("tgbm.model", param, model, dataset);
    std::vector<float> model_labels = dataset.label;
    dataset.load_from_file(param.path, param);
    if (!objective_needs_group_label(param.objective)) dataset.label = model_labels;
    std::vector<float> y_pred = predict(param, model, dataset, true);
    (void)y_pred;
    return 0;
}
