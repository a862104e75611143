// BatchedComputeKernel: the object a Glinthawk worker talks to (compute/kernel.hh).  States are
// pushed from the worker's thread; a bookkeeping thread binds each one to its context slots
// (PreallocatingContextManager::get_contexts, under the manager's mutex), an execution thread runs
// Model::forward() on it, and the finished state appears in the outgoing queue while an eventfd is
// signalled so that the worker's poll loop wakes up (compute/kernel.hh:103-170).
//
//   push( state&& )   any thread; never blocks on the GPU
//   pop( state& )     false when nothing has finished yet
//   event_fd()        non-semaphore eventfd: one read returns and clears the number of states
//                     finished since the last read (util/eventfd.hh)
//
// States leave in the order they were pushed: both stages are single threads with FIFO queues.
// A batch for which the manager has no room aborts -- the reference dereferences the empty optional
// there (kernel.hh:66-72): the router upstream is supposed to have reserved the space.
#pragma once

#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <queue>
#include <stop_token>
#include <sys/eventfd.h>
#include <thread>
#include <unistd.h>
#include <utility>
#include <vector>

#include "glint/contextman.hh"
#include "glint/state.hh"
#include "glint/types.hh"

namespace glint {

class EventFD
{
  int fd_ { -1 };

public:
  explicit EventFD( const bool semaphore = false )
    : fd_( ::eventfd( 0u, ( semaphore ? EFD_SEMAPHORE : 0 ) | EFD_NONBLOCK ) )
  {
    if ( fd_ < 0 ) {
      fatal( __FILE__, __LINE__, "eventfd:", std::strerror( errno ) );
    }
  }
  EventFD( const EventFD& ) = delete;
  EventFD& operator=( const EventFD& ) = delete;
  ~EventFD()
  {
    if ( fd_ >= 0 ) {
      ::close( fd_ );
    }
  }

  int fd_num() const { return fd_; }

  // false when there was nothing to read; `count` (optional) receives the counter that was cleared
  bool read_event( uint64_t* count = nullptr )
  {
    uint64_t value = 0;
    const ssize_t n = ::read( fd_, &value, sizeof( value ) );
    if ( n == (ssize_t)sizeof( value ) ) {
      if ( count != nullptr ) {
        *count = value;
      }
      return true;
    }
    if ( n < 0 && errno == EAGAIN ) {
      return false;
    }
    fatal( __FILE__, __LINE__, "eventfd_read:", std::strerror( errno ) );
  }

  void write_event()
  {
    const uint64_t value = 1;
    if ( ::write( fd_, &value, sizeof( value ) ) < 0 ) {
      fatal( __FILE__, __LINE__, "eventfd_write:", std::strerror( errno ) );
    }
  }
};

template<typename Model>
class BatchedComputeKernel
{
public:
  using ModelConfig = typename Model::ConfigType;
  using BatchedState = BatchedInferenceState<ModelConfig>;
  using ContextPtr = std::shared_ptr<typename Model::ContextType>;

  template<typename... Args>
  explicit BatchedComputeKernel( Args&&... args )
    : model_( std::make_unique<Model>( std::forward<Args>( args )... ) )
    , context_manager_( std::make_unique<PreallocatingContextManager<Model>>( model_->settings() ) )
    , execution_thread_( [this]( std::stop_token st ) { execution_loop( st ); } )
    , bookkeeping_thread_( [this]( std::stop_token st ) { bookkeeping_loop( st ); } )
  {
  }

  // the threads are asked to stop and joined (members are destroyed in reverse order: threads first)
  ~BatchedComputeKernel() = default;

  void push( BatchedState&& state )
  {
    {
      std::lock_guard lock( incoming_mutex_ );
      incoming_.push( std::move( state ) );
    }
    incoming_cv_.notify_one();
  }

  bool pop( BatchedState& state )
  {
    std::lock_guard lock( outgoing_mutex_ );
    if ( outgoing_.empty() ) {
      return false;
    }
    state = std::move( outgoing_.front() );
    outgoing_.pop();
    return true;
  }

  EventFD& event_fd() { return event_fd_; }
  Model& model() { return *model_; }
  PreallocatingContextManager<Model>& context_manager() { return *context_manager_; }

private:
  void bookkeeping_loop( std::stop_token stoken )
  {
    while ( !stoken.stop_requested() ) {
      BatchedState state;
      {
        std::unique_lock lock( incoming_mutex_ );
        if ( !incoming_cv_.wait( lock, stoken, [this] { return !incoming_.empty(); } ) ) {
          continue; // woken by the stop request
        }
        state = std::move( incoming_.front() );
        incoming_.pop();
      }
      auto contexts = context_manager_->get_contexts( state );
      if ( !contexts.has_value() ) {
        fatal( __FILE__, __LINE__, "BatchedComputeKernel:", "no context space for a batch the router has admitted" );
      }
      {
        std::lock_guard lock( processing_mutex_ );
        processing_.emplace( std::move( state ), std::move( *contexts ) );
      }
      processing_cv_.notify_one();
    }
  }

  void execution_loop( std::stop_token stoken )
  {
    while ( !stoken.stop_requested() ) {
      std::pair<BatchedState, std::vector<ContextPtr>> work;
      {
        std::unique_lock lock( processing_mutex_ );
        if ( !processing_cv_.wait( lock, stoken, [this] { return !processing_.empty(); } ) ) {
          continue;
        }
        work = std::move( processing_.front() );
        processing_.pop();
      }
      model_->forward( work.first, work.second );
      {
        std::lock_guard lock( outgoing_mutex_ );
        outgoing_.push( std::move( work.first ) );
      }
      event_fd_.write_event();
    }
  }

  std::unique_ptr<Model> model_;
  std::unique_ptr<PreallocatingContextManager<Model>> context_manager_;

  std::queue<BatchedState> incoming_ {}, outgoing_ {};
  std::queue<std::pair<BatchedState, std::vector<ContextPtr>>> processing_ {};
  std::mutex incoming_mutex_ {}, processing_mutex_ {}, outgoing_mutex_ {};
  std::condition_variable_any incoming_cv_ {}, processing_cv_ {};
  EventFD event_fd_ {};

  // last members: destroyed (stopped and joined) before anything they use
  std::jthread execution_thread_;
  std::jthread bookkeeping_thread_;
};

} // namespace glint
