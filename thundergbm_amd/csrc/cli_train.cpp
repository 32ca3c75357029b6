// thundergbm-train: parse a key=value config (plus argv overrides), load LIBSVM data, train, write
// "tgbm.model" (the reference's src/thundergbm/thundergbm_train.cpp).
#include "host.h"

using namespace tgbm;

int main(int argc, char **argv) {
    GBMParam param;
    Parser::parse_param(param, argc, argv);
    g_verbose = param.verbose;
    DataSet dataset;
    dataset.load_from_file(param.path, param);
    std::vector<std::vector<Tree>> model = train(param, dataset);
    Parser::save_model("tgbm.model", param, model, dataset);
    return 0;
}
