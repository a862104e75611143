// Context-slot bookkeeping: `max_context_count` contexts are created up front and handed out on
// first use of a context id; ids are sticky, so a finished prompt's slot is reused in place by the
// prompt that inherits its id.  Same rules as the reference's PreallocatingContextManager
// (compute/contextman.hh:56-196):
//   - free slots form a FIFO, the front is taken on allocation
//   - get_contexts() is two-phase: first count the active rows whose id is unmapped (duplicates
//     count each time); if more than free(), nothing is allocated and nullopt is returned
//   - inactive rows get the shared *empty* context
// release_context() follows the code after the reference's abort (tail of the FIFO), and is an
// extension here: the reference never releases.
#pragma once

#include <list>
#include <memory>
#include <mutex>
#include <optional>
#include <unordered_map>
#include <vector>

#include "glint/state.hh"
#include "glint/types.hh"

namespace glint {

template<typename Model>
class PreallocatingContextManager
{
public:
  using StateType = BatchedInferenceState<typename Model::ConfigType>;
  using ContextPtr = std::shared_ptr<typename Model::ContextType>;

  explicit PreallocatingContextManager( const typename Model::SettingsType& settings )
    : empty_context_( std::make_shared<typename Model::ContextType>( settings, true ) )
  {
    for ( size_t i = 0; i < settings.max_context_count; i++ ) {
      free_contexts_.emplace_back( std::make_shared<typename Model::ContextType>( settings ) );
      slot_of_[free_contexts_.back().get()] = static_cast<int32_t>( i );
    }
  }

  // single lookup (the deprecated path of the reference): null pointer when exhausted
  ContextPtr get_context( const ContextID& context_id )
  {
    std::lock_guard lock { mutex_ };
    if ( auto it = allocated_contexts_.find( context_id ); it != allocated_contexts_.end() ) {
      return it->second;
    }
    if ( free_contexts_.empty() ) {
      return {};
    }
    return take_front( context_id );
  }

  std::optional<std::vector<ContextPtr>> get_contexts( const StateType& state, const size_t start_ind, const size_t end_ind )
  {
    std::vector<ContextPtr> contexts;
    contexts.reserve( end_ind - start_ind );
    std::lock_guard lock { mutex_ };

    size_t missing = 0;
    for ( size_t i = start_ind; i < end_ind; i++ ) {
      if ( state.active( i ) && allocated_contexts_.find( state.context_id( i ) ) == allocated_contexts_.end() ) {
        missing++;
      }
    }
    if ( missing > free_contexts_.size() ) {
      return std::nullopt;
    }
    for ( size_t i = start_ind; i < end_ind; i++ ) {
      if ( !state.active( i ) ) {
        contexts.push_back( empty_context_ );
      } else if ( auto it = allocated_contexts_.find( state.context_id( i ) ); it != allocated_contexts_.end() ) {
        contexts.push_back( it->second );
      } else {
        contexts.push_back( take_front( state.context_id( i ) ) );
      }
    }
    return contexts;
  }

  std::optional<std::vector<ContextPtr>> get_contexts( const StateType& state ) { return get_contexts( state, 0, state.batch_size() ); }

  bool release_context( const ContextID& context_id )
  {
    std::lock_guard lock { mutex_ };
    auto it = allocated_contexts_.find( context_id );
    if ( it == allocated_contexts_.end() ) {
      return false;
    }
    free_contexts_.push_back( std::move( it->second ) );
    allocated_contexts_.erase( it );
    return true;
  }

  [[nodiscard]] size_t free() const { return free_contexts_.size(); }
  [[nodiscard]] size_t allocated() const { return allocated_contexts_.size(); }
  [[nodiscard]] size_t total() const { return free() + allocated(); }

  // creation index of a context (-1 for the shared empty context): what the parity tests compare
  int32_t slot_index( const ContextPtr& ctx ) const
  {
    auto it = slot_of_.find( ctx.get() );
    return it == slot_of_.end() ? -1 : it->second;
  }

private:
  ContextPtr take_front( const ContextID& context_id )
  {
    auto [it, inserted] = allocated_contexts_.emplace( context_id, std::move( free_contexts_.front() ) );
    free_contexts_.pop_front();
    return it->second;
  }

  std::mutex mutex_ {};
  std::list<ContextPtr> free_contexts_ {};
  const ContextPtr empty_context_;
  std::unordered_map<ContextID, ContextPtr> allocated_contexts_ {};
  std::unordered_map<const void*, int32_t> slot_of_ {};
};

} // namespace glint
