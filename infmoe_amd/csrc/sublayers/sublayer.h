// The expert ("sub-layer") plug-in point is public: include/infmoe_sublayer.h declares MoESubLayer,
// GroupedRun, RowTile and register_sublayer.  This header adds what the layer itself needs of it.
#pragma once

#include <memory>

#include "../../../include/infmoe_sublayer.h"
#include "../kernels/kernels.h"
#include "../status.h"

namespace infmoe {

// Replaces MoELayerPlugin::createSublayer (plugin/MoELayerPlugin.cc:28-41): looks `type` up among the
// registered factories ("T5_FF", "Identity" and whatever register_sublayer added).
Status make_sublayer(const char* type, const SubLayerConfig& config, std::shared_ptr<MoESubLayer>* out);

}  // namespace infmoe
