// SPDX-License-Identifier: Apache-2.0
/**
 * @file   nntr_api.h
 * @brief  The framework API the HIP plug-in is written against.
 *
 * Built inside the framework's tree (HIPQ_WITH_NNTRAINER defined, the
 * framework's include directories on the command line) this pulls in the real
 * headers; anywhere else it pulls in the stand-in that declares the same names.
 */
#ifndef NNTR_API_H
#define NNTR_API_H

#ifdef HIPQ_WITH_NNTRAINER
#include <context.h>
#include <layer.h>
#include <layer_context.h>
#include <layer_devel.h>
#include <mem_allocator.h>
#include <nntrainer_error.h>
#include <tensor.h>
#include <tensor_dim.h>
#else
#include "nntr_api_mirror.h"
#endif

#endif /* NNTR_API_H */
