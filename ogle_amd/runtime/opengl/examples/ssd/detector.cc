#include "opengl/examples/ssd/detector.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>

#include "ogle_hip.h"
#include "opengl/core/fbo_session.h"
#include "opengl/core/tensor.h"

namespace opengl {

std::unique_ptr<Detector> Detector::Create(const DetectorOptions& options) {
  FBOSession* session = new FBOSession;
  session->LoadGraph(options.model_name);
  return std::unique_ptr<Detector>(new Detector(session, true, options));
}

std::unique_ptr<Detector> Detector::Create(FBOSession* session, const DetectorOptions& options) {
  return std::unique_ptr<Detector>(new Detector(session, false, options));
}

Detector::Detector(FBOSession* session, bool owned, const DetectorOptions& options)
    : options_(options), session_(session), owns_session_(owned) {
  CHECK_EQ(options_.variances.size(), 4u);
  CHECK_EQ(options_.output_names.size(), 3u);
  CHECK_GE(options_.input_names.size(), 1u);
}

Detector::~Detector() {
  if (final_host_ != nullptr) (void)hipHostFree(final_host_);
  if (owns_session_) delete session_;
}

void Detector::Run(const Tensor* images) {
  session_->Run({{options_.input_names[0], const_cast<Tensor*>(images)}});
}

// Decode (decoder.glsl via functor::SSDBBoxDecoder, detector.cc:258) and the score
// filter of GenerateBoxInfo (detector.cc:184-225) in one device launch, then one
// readback of the compacted results.
void Detector::LoadToOutputTensors(const TensorNameList& names, int raw_width, int raw_height) {
  EnqueuePostprocess(names, raw_width, raw_height);
  Readback();
}

void Detector::EnqueuePostprocess(const TensorNameList& names, int raw_width, int raw_height,
                                  bool lists_in_place) {
  lists_in_place_ = lists_in_place;
  CHECK_EQ(names.size(), 3u);
  Tensor* cls_logits = session_->FindTensorByName(names[0]);
  Tensor* box_preds = session_->FindTensorByName(names[1]);
  Tensor* anchors = session_->FindTensorByName(names[2]);
  CHECK(cls_logits && box_preds && anchors) << "detector outputs were not produced";
  CHECK(cls_logits->outer_stride_bytes() == 0 && box_preds->outer_stride_bytes() == 0 &&
        anchors->outer_stride_bytes() == 0)
      << "the detector reads dense tensors: a head placed inside a concatenation cannot be named";
  CHECK_EQ(cls_logits->shape().size(), 3u);
  CHECK_EQ(box_preds->shape().size(), 3u);
  const int batch = box_preds->shape()[0], priors = box_preds->shape()[1];
  priors_for_nms_ = priors;
  const int classes = cls_logits->shape()[2];
  CHECK_EQ(box_preds->shape()[2], 4);
  CHECK_EQ(cls_logits->shape()[0], batch);
  CHECK_EQ(cls_logits->shape()[1], priors);
  CHECK_EQ(anchors->num_elements() % (static_cast<size_t>(priors) * 4), 0u);
  const size_t anchor_sets = anchors->num_elements() / (static_cast<size_t>(priors) * 4);
  CHECK(anchor_sets == 1 || anchor_sets == static_cast<size_t>(batch)) << "anchor shape";

  if (batch != batch_ || priors != priors_ || classes != classes_) {
    batch_ = batch; priors_ = priors; classes_ = classes;
    final_topk_ = 0;
    auto dev = [](IntList shape) {
      return std::unique_ptr<Tensor>(
          new Tensor(Tensor::DT_FLOAT, shape, Tensor::DEVICE_BUFFER, dlxnet::TensorProto::ANY4));
    };
    boxes_dev_ = dev({batch, priors, 4});
    count_dev_ = dev({batch});
    prior_dev_ = dev({batch, priors});
    class_dev_ = dev({batch, priors});
    score_dev_ = dev({batch, priors});
    box_dev_ = dev({batch, priors, 4});
    rect_dev_ = dev({batch, priors, 4});
    count_.resize(batch);
    prior_.resize(static_cast<size_t>(batch) * priors);
    class_.resize(prior_.size());
    score_.resize(prior_.size());
    box_.resize(prior_.size() * 4);
    rect_.resize(prior_.size() * 4);
  }
  OgleDetectArgs a{};
  a.logits_dev = static_cast<const float*>(cls_logits->device_ptr());
  a.prediction_dev = static_cast<const float*>(box_preds->device_ptr());
  a.anchors_dev = static_cast<const float*>(anchors->device_ptr());
  a.boxes_dev = static_cast<float*>(boxes_dev_->device_ptr());
  a.batch = batch; a.priors = priors; a.classes = classes;
  a.anchors_batch_stride = anchor_sets == 1 ? 0 : static_cast<int64_t>(priors) * 4;
  for (int i = 0; i < 4; ++i) a.variances[i] = options_.variances[i];
  a.score_threshold = options_.score_threshold;
  a.image_width = static_cast<float>(raw_width);
  a.image_height = static_cast<float>(raw_height);
  // in place: no compaction launch; only the device top-k + NMS can read such lists
  a.kept_count_dev = lists_in_place ? nullptr : static_cast<int32_t*>(count_dev_->device_ptr());
  a.kept_prior_dev = static_cast<int32_t*>(prior_dev_->device_ptr());
  a.kept_class_dev = static_cast<int32_t*>(class_dev_->device_ptr());
  a.kept_score_dev = static_cast<float*>(score_dev_->device_ptr());
  a.kept_box_dev = static_cast<float*>(box_dev_->device_ptr());
  a.kept_rect_dev = static_cast<int32_t*>(rect_dev_->device_ptr());
  session_->context()->Flush();
  hipStream_t s = static_cast<hipStream_t>(session_->context()->stream());
  const int64_t before = ogle_hip_launch_count();
  const int32_t st = ogle_hip_ssd_detect(&a, s);
  if (st != OGLE_OK) LOG(FATAL) << "ogle_hip_ssd_detect: " << ogle_hip_last_error();
  session_->context()->LogLaunches("detector.score_filter#Detector#", before);
}

void Detector::Readback() {
  CHECK(batch_ > 0) << "EnqueuePostprocess first";
  CHECK(!lists_in_place_) << "the kept lists were left in place for the device top-k + NMS";
  hipStream_t s = static_cast<hipStream_t>(session_->context()->stream());
  auto back = [&](void* dst, const Tensor* src, size_t bytes) {
    const hipError_t e = hipMemcpyAsync(dst, src->device_ptr(), bytes, hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) LOG(FATAL) << "readback: " << hipGetErrorString(e);
  };
  back(count_.data(), count_dev_.get(), count_.size() * 4);
  back(prior_.data(), prior_dev_.get(), prior_.size() * 4);
  back(class_.data(), class_dev_.get(), class_.size() * 4);
  back(score_.data(), score_dev_.get(), score_.size() * 4);
  back(box_.data(), box_dev_.get(), box_.size() * 4);
  back(rect_.data(), rect_dev_.get(), rect_.size() * 4);
  session_->context()->Finish();
}

namespace {
// One BoxInfo from entry `s` of the (prior, class, score, box, rect) arrays
// (detector.cc:211-225).
BoxInfo MakeBoxInfo(size_t s, const int32_t* prior, const int32_t* cls, const float* score,
                    const float* box, const int32_t* rect) {
  BoxInfo info;
  const float xmin = box[s * 4 + 0], ymin = box[s * 4 + 1];
  const float xmax = box[s * 4 + 2], ymax = box[s * 4 + 3];
  info.box.x = rect[s * 4 + 0];
  info.box.y = rect[s * 4 + 1];
  info.box.width = rect[s * 4 + 2];
  info.box.height = rect[s * 4 + 3];
  info.cx = static_cast<float>((xmin + xmax) / 2.0);
  info.cy = static_cast<float>((ymin + ymax) / 2.0);
  info.height = static_cast<float>(info.box.height);  // detector.cc:220-221
  info.width = static_cast<float>(info.box.width);
  info.score = score[s];
  info.class_name = cls[s];
  info.index = prior[s];
  return info;
}
}  // namespace

void Detector::GenerateBoxInfo(int image, std::vector<BoxInfo>* box_infos) const {
  CHECK(image >= 0 && image < batch_);
  box_infos->clear();
  const size_t base = static_cast<size_t>(image) * priors_;
  for (int r = 0; r < count_[image]; ++r)
    box_infos->push_back(MakeBoxInfo(base + r, prior_.data(), class_.data(), score_.data(), box_.data(),
                                     rect_.data()));
}

bool Detector::UsesDeviceNms() const {
  // the device kernel stages one image's scores and candidates in 64 KB of LDS
  const int priors = priors_for_nms_;
  return options_.device_nms && options_.topk >= 1 && options_.topk <= 1024 && priors <= 8192 &&
         4L * priors + 28L * options_.topk + 2048 <= 64 * 1024;
}

// Everything Detect does on the device after the network: with device top-k + NMS the
// score filter leaves its lists in place (no compaction launch) and the top-k + NMS
// launch reads them there; without, the score filter compacts them for the host.
void Detector::EnqueueDetect(const TensorNameList& names, int raw_width, int raw_height) {
  // whether the device kernel fits depends on the output shapes: look before launching
  const Tensor* box_preds = session_->FindTensorByName(names.size() == 3 ? names[1] : "");
  CHECK(box_preds != nullptr && box_preds->shape().size() == 3u) << "detector outputs were not produced";
  priors_for_nms_ = box_preds->shape()[1];
  const bool device = UsesDeviceNms();
  EnqueuePostprocess(names, raw_width, raw_height, device);
  if (device) EnqueueTopkNms();
}

void Detector::EnqueueTopkNms() {
  CHECK(batch_ > 0) << "EnqueuePostprocess first";
  const int topk = options_.topk;
  if (final_topk_ != topk) {
    if (final_host_ != nullptr) {   // sized for other lists: made anew below
      (void)hipHostFree(final_host_);
      final_host_ = nullptr;
    }
    final_topk_ = topk;
    final_dev_.reset(new Tensor(Tensor::DT_FLOAT, {static_cast<int>(FinalWords())}, Tensor::DEVICE_BUFFER,
                                dlxnet::TensorProto::ANY));
    final_staging_.assign(FinalWords(), 0);
  }
  if (want_host_copy_ && final_host_ == nullptr) {
    const hipError_t e = hipHostMalloc(&final_host_, FinalWords() * 4, hipHostMallocDefault);
    if (e != hipSuccess) LOG(FATAL) << "hipHostMalloc(" << FinalWords() * 4 << "): " << hipGetErrorString(e);
  }
  // where the six lists lie inside the block
  int32_t* const blk = static_cast<int32_t*>(final_dev_->device_ptr());
  const size_t bt = static_cast<size_t>(batch_) * topk;
  OgleNmsArgs a{};
  a.kept_count_dev =
      lists_in_place_ ? nullptr : static_cast<const int32_t*>(count_dev_->device_ptr());
  a.kept_prior_dev = static_cast<const int32_t*>(prior_dev_->device_ptr());
  a.kept_class_dev = static_cast<const int32_t*>(class_dev_->device_ptr());
  a.kept_score_dev = static_cast<const float*>(score_dev_->device_ptr());
  a.kept_box_dev = static_cast<const float*>(box_dev_->device_ptr());
  a.kept_rect_dev = static_cast<const int32_t*>(rect_dev_->device_ptr());
  a.batch = batch_;
  a.stride = priors_;
  a.topk = topk;
  a.nms_threshold = options_.nms_threshold;
  a.final_count_dev = blk;
  a.final_prior_dev = blk + batch_;
  a.final_class_dev = blk + batch_ + bt;
  a.final_score_dev = reinterpret_cast<float*>(blk + batch_ + 2 * bt);
  a.final_box_dev = reinterpret_cast<float*>(blk + batch_ + 3 * bt);
  a.final_rect_dev = blk + batch_ + 7 * bt;
  hipStream_t s = static_cast<hipStream_t>(session_->context()->stream());
  const int64_t before = ogle_hip_launch_count();
  const int32_t st = ogle_hip_ssd_topk_nms(&a, s);
  if (st != OGLE_OK) LOG(FATAL) << "ogle_hip_ssd_topk_nms: " << ogle_hip_last_error();
  session_->context()->LogLaunches("detector.topk_nms#Detector#", before);
  if (final_host_ != nullptr) {
    const hipError_t e =
        hipMemcpyAsync(final_host_, final_dev_->device_ptr(), FinalWords() * 4, hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) LOG(FATAL) << "copy of the final lists: " << hipGetErrorString(e);
  }
}

size_t Detector::FinalWords() const {
  return static_cast<size_t>(batch_) * (1 + static_cast<size_t>(final_topk_) * 11);
}

void Detector::EnableHostCopy() { want_host_copy_ = true; }

void Detector::ParseFinal(const int32_t* blk, std::vector<std::vector<BoxInfo>>* final_boxes) const {
  const size_t bt = static_cast<size_t>(batch_) * final_topk_;
  const int32_t* prior = blk + batch_;
  const int32_t* cls = prior + bt;
  const float* score = reinterpret_cast<const float*>(cls + bt);
  const float* box = score + bt;
  const int32_t* rect = reinterpret_cast<const int32_t*>(box + 4 * bt);
  final_boxes->assign(batch_, {});
  for (int b = 0; b < batch_; ++b) {
    const size_t base = static_cast<size_t>(b) * final_topk_;
    const int n = std::min(std::max(blk[b], 0), final_topk_);
    (*final_boxes)[b].reserve(n);
    for (int r = 0; r < n; ++r)
      (*final_boxes)[b].push_back(MakeBoxInfo(base + r, prior, cls, score, box, rect));
  }
}

void Detector::FinalFromHostCopy(std::vector<std::vector<BoxInfo>>* final_boxes) const {
  CHECK(final_host_ != nullptr && final_topk_ > 0) << "EnableHostCopy, then a pass with the detector's work";
  ParseFinal(static_cast<const int32_t*>(final_host_), final_boxes);
}

void Detector::ReadbackFinal(std::vector<std::vector<BoxInfo>>* final_boxes) {
  CHECK(final_topk_ > 0) << "EnqueueTopkNms first";
  hipStream_t s = static_cast<hipStream_t>(session_->context()->stream());
  const hipError_t e = hipMemcpyAsync(final_staging_.data(), final_dev_->device_ptr(), FinalWords() * 4,
                                      hipMemcpyDeviceToHost, s);
  if (e != hipSuccess) LOG(FATAL) << "readback: " << hipGetErrorString(e);
  session_->context()->Finish();
  ParseFinal(final_staging_.data(), final_boxes);
}

// detector.cc:114-125.  std::stable_sort makes the order of equal scores defined
// (ascending prior index); the reference's std::sort leaves it unspecified.
void Detector::GetTopK(std::vector<BoxInfo>& input, int top_k) {
  std::stable_sort(input.begin(), input.end(),
                   [](const BoxInfo& a, const BoxInfo& b) { return a.score > b.score; });
  if (top_k < static_cast<int>(input.size())) input.erase(input.begin() + top_k, input.end());
}

// detector.cc:127-148: j is dropped if ANY earlier i overlaps it, dropped or not.
void Detector::NMS(std::vector<BoxInfo>& boxes, std::vector<BoxInfo>& boxes_left, float threshold) {
  const int n = static_cast<int>(boxes.size());
  std::vector<int> labels(n, -1);
  for (int i = 0; i < n - 1; ++i)
    for (int j = i + 1; j < n; ++j)
      if (iou(boxes[i].box, boxes[j].box) > threshold) labels[j] = 0;
  for (int i = 0; i < n; ++i)
    if (labels[i] == -1) boxes_left.push_back(boxes[i]);
}

void Detector::Detect(const Tensor* images, int raw_width, int raw_height,
                      std::vector<std::vector<BoxInfo>>* final_boxes) {
  Run(images);
  EnqueueDetect(options_.output_names, raw_width, raw_height);
  if (UsesDeviceNms()) {
    ReadbackFinal(final_boxes);
    return;
  }
  Readback();
  HostTopkNms(final_boxes);
}

void Detector::HostTopkNms(std::vector<std::vector<BoxInfo>>* final_boxes) const {
  final_boxes->assign(batch_, {});
  for (int b = 0; b < batch_; ++b) {
    std::vector<BoxInfo> infos;
    GenerateBoxInfo(b, &infos);
    GetTopK(infos, options_.topk);
    NMS(infos, (*final_boxes)[b], options_.nms_threshold);
  }
}

// examples/ssd/common.cc:57-77.
float iou(const Rect& box0, const Rect& box1) {
  const float xmin0 = box0.x, ymin0 = box0.y;
  const float xmax0 = box0.x + box0.width, ymax0 = box0.y + box0.height;
  const float xmin1 = box1.x, ymin1 = box1.y;
  const float xmax1 = box1.x + box1.width, ymax1 = box1.y + box1.height;
  const float w = std::fmax(0.0f, std::fmin(xmax0, xmax1) - std::fmax(xmin0, xmin1));
  const float h = std::fmax(0.0f, std::fmin(ymax0, ymax1) - std::fmax(ymin0, ymin1));
  const float i = w * h;
  const float u = (xmax0 - xmin0) * (ymax0 - ymin0) + (xmax1 - xmin1) * (ymax1 - ymin1) - i;
  if (u <= 0.0) return 0.0f;
  return i / u;
}

}  // namespace opengl
